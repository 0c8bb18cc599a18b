// Fused GPTDecoder path: model object, weight loading/packing, prefill, decode step, on-device token loop.
//
// Replaces, for one model replica on one GPU, the reference's per-step stack
//   GPT.RunForwardOnSingleDevice      Seq2SeqSharp/Applications/GPT.cs:212-335
//   Decoder.GPTDecode                 Seq2SeqSharp/Applications/Decoder.cs:648-794
//   GPTDecoder.Decode                 Seq2SeqSharp/Networks/GPTDecoder.cs:153-191
//   GroupQueryAttention.Perform       Seq2SeqSharp/Layers/GroupQueryAttention.cs:114-233
//   MultiHeadAttention.PerformClassic Seq2SeqSharp/Layers/MultiHeadAttention.cs:125-240
//   PositionwiseFeedForward.Process   Seq2SeqSharp/Layers/PositionwiseFeedForward.cs:72-98
// with a preallocated compact KV cache instead of concat-and-reallocate, and with only token ids
// crossing PCIe per step.
#include "tship_gpt_kernels.h"
#include "tship_moe_kernels.h"
#include "tship_sample_kernels.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cxxabi.h>
#include <cstring>
#include <map>
#include <memory>
#include <set>
#include <vector>

namespace tship {

struct DevBuf {
    void* p = nullptr;
    size_t bytes = 0;
    void alloc(size_t b) {
        release();
        if (b == 0) b = 256;
        p = device_malloc_retry(b);      // (throws when the memory is not there even after the pool's cached blocks went back)
        bytes = b;
        TSHIP_CHECK_HIP(hipMemsetAsync(p, 0, b, stream()));
    }
    void release() {
        if (p) { (void)hipStreamSynchronize(stream()); (void)hipFree(p); p = nullptr; bytes = 0; }
    }
    // grow-only workspace: keeps the allocation (and its contents) when it is already large enough
    void reserve(size_t b) { if (b > bytes) alloc(b); }
    ~DevBuf() { release(); }
    DevBuf() {}
    DevBuf(const DevBuf&) = delete;
    DevBuf& operator=(const DevBuf&) = delete;
    template <typename T> T* as() const { return (T*)p; }
};

// one GEMM operand: fp16 packed (KT x NT tiles) or fp32 row-major
struct GemmW {
    DevBuf buf;
    int K = 0, N = 0;      // logical
    int KT = 0, NT = 0;    // fp16 packed tile counts
    long ld = 0;           // fp32 leading dimension
    int KS = 1;            // split-K factor used at decode
};

struct LayerW {
    DevBuf n1_g, n1_b, n2_g, n2_b;
    GemmW qkv, wo, w13, w2;
    DevBuf bqkv, bo, b1, b3, b2;
    DevBuf kc, vc;
    // deferred LayerNorm: per packed output column the folded constants d (norm's beta through the weights, plus the bias)
    // followed by c (norm's gamma through the weights); see SkinnyArgs.  qkv: [2][round_up(Nqkv, 32)], w13: [2][NT * 32]
    DevBuf ln_qkv, ln_13;
    bool moe = false;
    // MoE (Seq2SeqSharp/Layers/MoEFeedForward.cs:49-55)
    DevBuf router, router_b;               // fp32 [h][E], [E]
    std::vector<std::unique_ptr<GemmW>> e1, e2;   // per expert [h][4h], [4h][h]
    DevBuf wtab1, wtab2;                   // device tables of the experts' weight pointers (fp16 decode GEMMs batch over them); written once at Finalize
    DevBuf route;                          // this layer's routing at the last step: probs [Bpad][E], top values [Bpad][k], top indices [Bpad][k]
};

// demangled name of the device function behind a __global__ host stub (what a profiler's kernel trace shows)
static std::string kernel_symbol(const void* host_fn) {
    const char* raw = hipKernelNameRefByPtr(host_fn, stream());
    if (!raw) { (void)hipGetLastError(); return std::string(); }
    int status = 0;
    char* dem = abi::__cxa_demangle(raw, nullptr, nullptr, &status);
    if (status != 0 || !dem) {
        // (this demangler does not know the _Float16 type code DF16_: spell it as the older half type Dh for the name's sake)
        std::free(dem); dem = nullptr;
        std::string alt(raw);
        for (size_t i = alt.find("DF16_"); i != std::string::npos; i = alt.find("DF16_", i)) alt.replace(i, 5, "Dh");
        dem = abi::__cxa_demangle(alt.c_str(), nullptr, nullptr, &status);
    }
    std::string out = (status == 0 && dem) ? dem : raw;
    std::free(dem);
    return out;
}

struct Profiler {
    std::vector<std::string> names, symbols;
    std::vector<hipEvent_t> ev0, ev1;
    ~Profiler() { for (auto e : ev0) (void)hipEventDestroy(e); for (auto e : ev1) (void)hipEventDestroy(e); }
};

}  // namespace tship

using namespace tship;

struct TSHipGpt {
    TSHipGptConfig c;
    bool f16;
    int D, G, Nqkv, Bpad, BT;      // G: query heads per block of the attention kernels (all of a KV head's, or a group of them)
    int SG = 1, Hv = 0;            // groups of G query heads per KV head (more than eight heads per KV head), and n_kv_heads * SG
    long ldh, ldF;                 // leading dims of activation buffers (elements)
    int F13;                       // columns of the first FFN GEMM output (F or 2F)
    bool gated;
    std::vector<std::unique_ptr<LayerW>> L;
    DevBuf emb;                    // [V][h] model dtype
    DevBuf seg;                    // segment embeddings, fp32 [max_segments][h] (null without them); pw_seg: a prefill's segment of every row
    DevBuf pw_seg;
    DevBuf fn_g, fn_b;             // final norm
    GemmW head; DevBuf head_b;
    DevBuf rope_cos, rope_sin;
    std::set<std::string> expected, seen;
    bool finalized = false;

    // decode state
    DevBuf x, xn, o, a, part_qkv, part_h, part_f, logits, ids, d_pos, hidden;
    DevBuf moe_ws, topp_scratch, topp_uni, gen_buf, uni_buf, tile_count;
    DevBuf pw_lens, pw_ids, pw_x, pw_xn, pw_qkv, pw_o, pw_a, pw_f, pw_rowmap, pw_ssq, pw_rinv, pw_zero_bias, pw_moe;     // prefill workspace
    DevBuf ssq;                    // deferred-norm path: per-column-tile sums of squares [h/32][Bpad]
    bool fused_norm = false;       // fp16 + dense layers (RMSNorm; LayerNorm up to 32 rows): residual/norm folded into the GEMM tails
    bool ln = false;               // that path with LayerNorm: tile sums of x beside the sums of squares, folded constants per consumer
    DevBuf ln_head;                // [2][round_up(vocab, 32)]: d then c of the vocabulary projection behind the final norm
    bool vt = false;               // fp16 cache with head_dim 64/128: keys and values stored fragment-major for the MFMA attention kernels
    long ML = 0;                   // cache rows per (sequence, KV head): max_seq_len rounded up to 32
    // one decode step (sample + decode) captured as a HIP graph; valid for one (batch, sampling mode) at a time
    hipGraphExec_t step_graph = nullptr;
    int graph_batch = 0, graph_mode = -1; float graph_top_p = 0.0f, graph_temp = 0.0f;
    const float* graph_uniforms = nullptr; int* graph_gen = nullptr;
    int pos = 0;                   // host mirror of *d_pos
    // repeat penalty of top-p sampling (DecodingOptions.RepeatPenalty): last sequence index of every token, per sequence
    DevBuf last_pos; long last_ld = 0; float repeat_penalty = 0.0f; float graph_penalty = 0.0f;
    static constexpr int MAX_ATTN_SPLITS = 16;
    DevBuf attn_xchg, attn_count;  // decode attention with several blocks per (row, KV head): partial sums and one counter per pair
    bool any_blocked = false;
    bool embed_done = false;       // the sampling kernel of this step has already done the next step's embedding (greedy_embed_kernel)
    DevBuf blocked;                // one byte per token, non-zero = DecodingOptions.BlockedTokens (allocated with the model: graphs keep its address)
    int cur_batch = 0;
    std::vector<std::string> last_symbols;      // launched symbols of the last profiled step, in launch order
    DevBuf beam_probs, beam_ids, beam_out, beam_uni, reorder_tmp, reorder_src;      // beam search: probabilities the picks consume, picks, gather temporaries
    Profiler* prof = nullptr;

    size_t esz() const { return f16 ? 2 : 4; }
};

// A saved set of sequences: the used prefix of every (sequence, KV head) cache region of every layer, in the cache's own
// layout and element type, plus what a decode step afterwards needs (logits of the last step, token history).  Device
// memory only; TSHip_GptSaveRows fills it and TSHip_GptRestoreRows copies it back, device to device.
struct TSHipGptSnapshot {
    int batch = 0, len = 0;
    int n_layers = 0, n_kv_heads = 0, D = 0, vocab = 0; bool f16 = false, vt = false;
    size_t region_bytes = 0;                       // saved bytes per (sequence, KV head) region
    std::vector<std::unique_ptr<tship::DevBuf>> k, v;
    tship::DevBuf logits, last_pos; long last_ld = 0;
    size_t total_bytes = 0;
};

namespace tship {

// Test hooks (environment variables, listed in include/tship.h).  They are read once per call of an entry point that runs
// the model (refresh_test_hooks), never inside the per-layer code.
struct TestHooks {
    int ffn_tiles = 0;        // TSHIP_FFN_TILES: 10, 15, 20, 30 or 40 = column tiles x 10 per block of the decode FFN up projection
    int patch_rows = 0;       // TSHIP_PATCH_ROWS: 1, 2, 4 or 8 row tiles per tile patch of the prefill GEMM
    long attn_splits = 0;     // TSHIP_ATTN_SPLITS: blocks per (sequence, KV head) pair in decode attention
    int attn_nq = 0;          // TSHIP_ATTN_NQ: 1 or 2 groups of 16 MFMA columns per wavefront in prefill attention
    bool no_kv_fuse = false;  // TSHIP_NO_KV_FUSE: the QKV projection of a prefill does not write the cache itself
    bool no_moe_batch = false;// TSHIP_NO_MOE_BATCH: one prefill GEMM launch per expert
    bool no_graph = false;    // TSHIP_NO_GRAPH: the generate loop launches its kernels one by one
};
static TestHooks g_hooks;
static void refresh_test_hooks() {
    TestHooks h;
    if (const char* v = std::getenv("TSHIP_FFN_TILES")) {
        h.ffn_tiles = std::atoi(v);
        TSHIP_REQUIRE(h.ffn_tiles == 10 || h.ffn_tiles == 15 || h.ffn_tiles == 20 || h.ffn_tiles == 30 || h.ffn_tiles == 40, "TSHIP_FFN_TILES: 10, 15, 20, 30 or 40");
    }
    if (const char* v = std::getenv("TSHIP_PATCH_ROWS")) {
        h.patch_rows = std::atoi(v);
        TSHIP_REQUIRE(h.patch_rows == 1 || h.patch_rows == 2 || h.patch_rows == 4 || h.patch_rows == 8, "TSHIP_PATCH_ROWS: 1, 2, 4 or 8");
    }
    if (const char* v = std::getenv("TSHIP_ATTN_SPLITS")) { h.attn_splits = std::atol(v); TSHIP_REQUIRE(h.attn_splits >= 1, "TSHIP_ATTN_SPLITS: a positive number"); }
    if (const char* v = std::getenv("TSHIP_ATTN_NQ")) { h.attn_nq = std::atoi(v); TSHIP_REQUIRE(h.attn_nq == 1 || h.attn_nq == 2, "TSHIP_ATTN_NQ: 1 or 2"); }
    h.no_kv_fuse = std::getenv("TSHIP_NO_KV_FUSE") != nullptr;
    h.no_moe_batch = std::getenv("TSHIP_NO_MOE_BATCH") != nullptr;
    h.no_graph = std::getenv("TSHIP_NO_GRAPH") != nullptr;
    g_hooks = h;
}

template <typename... KArgs, typename... Args>
static void launch(TSHipGpt* m, const char* name, void (*kernel)(KArgs...), dim3 grid, dim3 block, Args... args) {
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (m && m->prof) {
        TSHIP_CHECK_HIP(hipEventCreate(&e0));
        TSHIP_CHECK_HIP(hipEventCreate(&e1));
        m->prof->names.push_back(name);
        m->prof->symbols.push_back(kernel_symbol((const void*)kernel));
        m->prof->ev0.push_back(e0);
        m->prof->ev1.push_back(e1);
    }
    if (e0) hipExtLaunchKernelGGL(kernel, grid, block, 0, stream(), e0, e1, 0, args...);
    else hipLaunchKernelGGL(kernel, grid, block, 0, stream(), args...);
    TSHIP_CHECK_HIP(hipGetLastError());
}

// launch with dynamic LDS beyond the 64 KiB default limit (the attribute is set once per kernel)
template <typename... KArgs, typename... Args>
static void launch_shm(TSHipGpt* m, const char* name, void (*kernel)(KArgs...), dim3 grid, dim3 block, unsigned shm, Args... args) {
    static std::map<const void*, unsigned> raised;
    unsigned& have = raised[(const void*)kernel];
    if (shm > 65536u && shm > have) {
        TSHIP_REQUIRE(shm <= 160u * 1024u, "dynamic LDS request exceeds the 160 KiB of a compute unit");
        TSHIP_CHECK_HIP(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm));
        have = shm;
    }
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (m && m->prof) {
        TSHIP_CHECK_HIP(hipEventCreate(&e0));
        TSHIP_CHECK_HIP(hipEventCreate(&e1));
        m->prof->names.push_back(name);
        m->prof->symbols.push_back(kernel_symbol((const void*)kernel));
        m->prof->ev0.push_back(e0);
        m->prof->ev1.push_back(e1);
    }
    if (e0) hipExtLaunchKernelGGL(kernel, grid, block, shm, stream(), e0, e1, 0, args...);
    else hipLaunchKernelGGL(kernel, grid, block, shm, stream(), args...);
    TSHIP_CHECK_HIP(hipGetLastError());
}

// decode GEMM launch: the scalars that the kernel's first requests depend on travel as leading arguments of their own
// (preloaded into scalar registers at wavefront start), the rest in the struct
template <typename... KArgs>
static void launch_skinny(TSHipGpt* m, const char* name, void (*kernel)(KArgs...), dim3 grid, dim3 block, const SkinnyArgs& e) {
    launch(m, name, kernel, grid, block, e.W, e.X, e.KT, e.NT, e.KS, e.rows_valid, e.ssq, e.ssq_nt, e.ssq_ld, e.ln, e);
}

// decode GEMM split-K: a block has NW wavefronts of 8 k-tiles each in flight; split K across blocks until one
// pass covers the block's range (keeps partial-sum traffic small: K = 2048 needs no split at batch <= 32)
static int pick_ks_f16(int NT, int KT, int BT) {
    const int NW = BT <= 2 ? 8 : 4;
    int ks = (int)ceil_div(KT, NW * 8);
    // few column tiles (small models): split further, up to one block per compute unit, while every wavefront keeps two
    // k-tiles (32 blocks that each walk the whole K are bound by one block's latency, not by bandwidth)
    const int fill = std::min(n_compute_units() / std::max(1, NT), KT / (NW * 2));
    ks = std::max(ks, fill);
    return std::max(1, std::min(ks, 16));
}
static int pick_ks_f32(int N, int K) {
    int target = 2 * std::max(n_compute_units(), 64);
    int ks = std::max(1, target / (int)ceil_div(N, 64));
    ks = std::min(ks, std::max(1, K / 64));
    return std::min(ks, 16);
}

static void upload_f32(DevBuf& dst, const float* host, size_t n) {
    dst.alloc(n * sizeof(float));
    TSHIP_CHECK_HIP(hipMemcpyAsync(dst.p, host, n * sizeof(float), hipMemcpyHostToDevice, stream()));
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
}

// allocate the destination of a GEMM weight with logical shape [K][N]
static void gemmw_alloc(TSHipGpt* m, GemmW& w, int K, int N) {
    if (w.buf.p) return;
    w.K = K; w.N = N;
    if (m->f16) {
        w.KT = (int)ceil_div(K, 16); w.NT = (int)ceil_div(N, 32);
        w.buf.alloc((size_t)w.KT * w.NT * 512 * sizeof(half_t));
        w.KS = pick_ks_f16(w.NT, w.KT, m->BT);
    } else {
        w.ld = N;
        w.buf.alloc((size_t)K * N * sizeof(float));
        w.KS = pick_ks_f32(N, K);
    }
}

// copy host fp32 [K][n_src] into columns of a GEMM weight (packing for fp16)
static void gemmw_fill(TSHipGpt* m, GemmW& w, const float* host, int K, int n_src, int mode, int n_off) {
    TSHIP_REQUIRE(K == w.K, "weight row count does not match the model configuration");
    DevBuf tmp;
    upload_f32(tmp, host, (size_t)K * n_src);
    if (m->f16) {
        long total = (long)n_src * w.KT * 2;
        pack_w_kernel<<<(unsigned)ceil_div(total, 256), 256, 0, stream()>>>(tmp.as<float>(), n_src, K, n_src, w.buf.as<half_t>(), w.KT, mode, n_off);
    } else {
        TSHIP_REQUIRE(mode == PACK_PLAIN, "internal: interleave is an fp16-only layout");
        long total = (long)K * n_src;
        copy_cols_kernel<float><<<(unsigned)ceil_div(total, 256), 256, 0, stream()>>>(tmp.as<float>(), n_src, K, n_src, w.buf.as<float>(), w.ld, n_off);
    }
    TSHIP_CHECK_HIP(hipGetLastError());
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
}

static void expect_shape(const char* name, int ndim, const int64_t* sizes, std::initializer_list<int64_t> want) {
    bool ok = (size_t)ndim == want.size();
    if (ok) { int i = 0; for (auto w : want) ok = ok && sizes[i++] == w; }
    if (!ok) {
        std::string s = std::string("weight '") + name + "' has shape [";
        for (int i = 0; i < ndim; ++i) s += (i ? "," : "") + std::to_string(sizes[i]);
        s += "], expected [";
        int i = 0; for (auto w : want) s += (i++ ? "," : "") + std::to_string(w);
        throw Error(s + "]");
    }
}

static void build_expected(TSHipGpt* m) {
    auto& c = m->c;
    auto& e = m->expected;
    bool ln = c.norm_type == 1;
    auto norm = [&](const std::string& p) { e.insert(p + ".m_alpha"); if (ln) e.insert(p + ".m_beta"); };
    e.insert("TgtEmbeddings");
    if (c.max_segments > 0) e.insert("SegmentEmbedding");
    for (int i = 0; i < c.n_layers; ++i) {
        std::string a = "GPTDecoder.SelfAttn_" + std::to_string(i);
        norm(a + ".layerNormQ");
        if (c.attn_type == 1) for (auto s : {"Q", "Qb", "K", "Kb", "V", "Vb"}) e.insert(a + "." + s);
        else { e.insert(a + ".QKV"); e.insert(a + ".QKVb"); }
        e.insert(a + ".W0"); e.insert(a + ".b0");
        if (c.n_experts > 1 && i > 1) {
            std::string f = "GPTDecoder.MoEFFN_" + std::to_string(i);
            for (auto s : {"layerNorm.m_alpha", "layerNorm.m_beta", "m_Router", "m_RouterBias", "m_Whd1", "m_Whd2"}) e.insert(f + "." + s);
        } else {
            std::string f = "GPTDecoder.PosFFN_" + std::to_string(i);
            norm(f + ".layerNorm2");
            e.insert(f + ".feedForwardLayer1.m_Whd"); e.insert(f + ".feedForwardLayer1.m_Bd");
            e.insert(f + ".feedForwardLayer2.m_Whd"); e.insert(f + ".feedForwardLayer2.m_Bd");
            if (m->gated) { e.insert(f + ".feedForwardLayer3.m_Whd"); e.insert(f + ".feedForwardLayer3.m_Bd"); }
        }
    }
    norm("GPTDecoder.layerNorm");
    e.insert("FeedForward_Decoder_0.m_Whd"); e.insert("FeedForward_Decoder_0.m_Bd");
}

static void set_weight(TSHipGpt* m, const std::string& name, const float* host, int ndim, const int64_t* sizes) {
    auto& c = m->c;
    TSHIP_REQUIRE(m->expected.count(name), "unknown weight name for this configuration: " + name);
    const int h = c.hidden, H = c.n_heads, Gk = c.n_kv_heads, D = m->D, F = c.ffn_dim, V = c.vocab;
    long count = 1; for (int i = 0; i < ndim; ++i) count *= sizes[i];
    auto vec = [&](DevBuf& dst, int64_t n) { expect_shape(name.c_str(), ndim, sizes, {1, n}); upload_f32(dst, host, (size_t)n); };
    auto vec_into = [&](DevBuf& dst, int64_t total, int64_t off, int64_t n) {
        expect_shape(name.c_str(), ndim, sizes, {1, n});
        if (!dst.p) dst.alloc((size_t)total * sizeof(float));
        TSHIP_CHECK_HIP(hipMemcpyAsync(dst.as<float>() + off, host, (size_t)n * sizeof(float), hipMemcpyHostToDevice, stream()));
        TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    };
    if (name == "TgtEmbeddings") {
        expect_shape(name.c_str(), ndim, sizes, {V, h});
        DevBuf tmp; upload_f32(tmp, host, (size_t)V * h);
        m->emb.alloc((size_t)V * h * m->esz());
        long total = (long)V * h;
        if (m->f16) copy_cols_kernel<half_t><<<(unsigned)ceil_div(total, 256), 256, 0, stream()>>>(tmp.as<float>(), h, V, h, m->emb.as<half_t>(), h, 0);
        else copy_cols_kernel<float><<<(unsigned)ceil_div(total, 256), 256, 0, stream()>>>(tmp.as<float>(), h, V, h, m->emb.as<float>(), h, 0);
        TSHIP_CHECK_HIP(hipGetLastError());
        TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    } else if (name == "SegmentEmbedding") {
        expect_shape(name.c_str(), ndim, sizes, {c.max_segments, h});
        upload_f32(m->seg, host, (size_t)c.max_segments * h);
    } else if (name == "GPTDecoder.layerNorm.m_alpha") vec(m->fn_g, h);
    else if (name == "GPTDecoder.layerNorm.m_beta") vec(m->fn_b, h);
    else if (name == "FeedForward_Decoder_0.m_Whd") {
        expect_shape(name.c_str(), ndim, sizes, {h, V});
        gemmw_alloc(m, m->head, h, V); m->head.KS = 1;
        gemmw_fill(m, m->head, host, h, V, PACK_PLAIN, 0);
    } else if (name == "FeedForward_Decoder_0.m_Bd") vec(m->head_b, V);
    else {
        // GPTDecoder.<kind>_<i>.<field>
        size_t us = name.find('_'), dot = name.find('.', us);
        TSHIP_REQUIRE(us != std::string::npos && dot != std::string::npos, "cannot parse weight name: " + name);
        int li = std::stoi(name.substr(us + 1, dot - us - 1));
        TSHIP_REQUIRE(li >= 0 && li < c.n_layers, "layer index out of range in weight name: " + name);
        LayerW& L = *m->L[li];
        std::string kind = name.substr(0, us), field = name.substr(dot + 1);
        if (kind == "GPTDecoder.SelfAttn") {
            if (field == "layerNormQ.m_alpha") vec(L.n1_g, h);
            else if (field == "layerNormQ.m_beta") vec(L.n1_b, h);
            else if (field == "QKV") { expect_shape(name.c_str(), ndim, sizes, {h, 3 * h}); gemmw_alloc(m, L.qkv, h, m->Nqkv); gemmw_fill(m, L.qkv, host, h, 3 * h, PACK_PLAIN, 0); }
            else if (field == "QKVb") vec(L.bqkv, 3 * h);
            else if (field == "Q") { expect_shape(name.c_str(), ndim, sizes, {h, H * D}); gemmw_alloc(m, L.qkv, h, m->Nqkv); gemmw_fill(m, L.qkv, host, h, H * D, PACK_PLAIN, 0); }
            else if (field == "K") { expect_shape(name.c_str(), ndim, sizes, {h, Gk * D}); gemmw_alloc(m, L.qkv, h, m->Nqkv); gemmw_fill(m, L.qkv, host, h, Gk * D, PACK_PLAIN, H * D); }
            else if (field == "V") { expect_shape(name.c_str(), ndim, sizes, {h, Gk * D}); gemmw_alloc(m, L.qkv, h, m->Nqkv); gemmw_fill(m, L.qkv, host, h, Gk * D, PACK_PLAIN, H * D + Gk * D); }
            else if (field == "Qb") vec_into(L.bqkv, m->Nqkv, 0, H * D);
            else if (field == "Kb") vec_into(L.bqkv, m->Nqkv, H * D, Gk * D);
            else if (field == "Vb") vec_into(L.bqkv, m->Nqkv, H * D + Gk * D, Gk * D);
            else if (field == "W0") { expect_shape(name.c_str(), ndim, sizes, {h, h}); gemmw_alloc(m, L.wo, h, h); gemmw_fill(m, L.wo, host, h, h, PACK_PLAIN, 0); }
            else if (field == "b0") vec(L.bo, h);
            else throw Error("unknown attention field: " + name);
        } else if (kind == "GPTDecoder.PosFFN") {
            bool inter = m->f16 && m->gated;     // fp16: W1/W3 interleaved by 16 columns; fp32: [W1 | W3]
            if (field == "layerNorm2.m_alpha") vec(L.n2_g, h);
            else if (field == "layerNorm2.m_beta") vec(L.n2_b, h);
            else if (field == "feedForwardLayer1.m_Whd") {
                expect_shape(name.c_str(), ndim, sizes, {h, F});
                gemmw_alloc(m, L.w13, h, m->F13); if (m->f16) L.w13.KS = 1;
                gemmw_fill(m, L.w13, host, h, F, inter ? PACK_INTERLEAVE16 : PACK_PLAIN, 0);
            } else if (field == "feedForwardLayer3.m_Whd") {
                expect_shape(name.c_str(), ndim, sizes, {h, F});
                gemmw_alloc(m, L.w13, h, m->F13); if (m->f16) L.w13.KS = 1;
                gemmw_fill(m, L.w13, host, h, F, inter ? PACK_INTERLEAVE16 : PACK_PLAIN, inter ? 16 : F);
            } else if (field == "feedForwardLayer1.m_Bd") vec(L.b1, F);
            else if (field == "feedForwardLayer3.m_Bd") vec(L.b3, F);
            else if (field == "feedForwardLayer2.m_Whd") { expect_shape(name.c_str(), ndim, sizes, {F, h}); gemmw_alloc(m, L.w2, F, h); gemmw_fill(m, L.w2, host, F, h, PACK_PLAIN, 0); }
            else if (field == "feedForwardLayer2.m_Bd") vec(L.b2, h);
            else throw Error("unknown feed-forward field: " + name);
        } else if (kind == "GPTDecoder.MoEFFN") {
            const int E = c.n_experts;
            if (field == "layerNorm.m_alpha") vec(L.n2_g, h);
            else if (field == "layerNorm.m_beta") vec(L.n2_b, h);
            else if (field == "m_Router") { expect_shape(name.c_str(), ndim, sizes, {h, E}); upload_f32(L.router, host, (size_t)h * E); }
            else if (field == "m_RouterBias") vec(L.router_b, E);
            else if (field == "m_Whd1") {
                expect_shape(name.c_str(), ndim, sizes, {E, h, 4 * h});
                for (int e = 0; e < E; ++e) { gemmw_alloc(m, *L.e1[e], h, 4 * h); L.e1[e]->KS = 1; gemmw_fill(m, *L.e1[e], host + (size_t)e * h * 4 * h, h, 4 * h, PACK_PLAIN, 0); }
            } else if (field == "m_Whd2") {
                expect_shape(name.c_str(), ndim, sizes, {E, 4 * h, h});
                for (int e = 0; e < E; ++e) { gemmw_alloc(m, *L.e2[e], 4 * h, h); L.e2[e]->KS = 1; gemmw_fill(m, *L.e2[e], host + (size_t)e * h * 4 * h, 4 * h, h, PACK_PLAIN, 0); }
            } else throw Error("unknown MoE field: " + name);
        } else throw Error("unknown weight name: " + name);
    }
    (void)count;
    m->seen.insert(name);
}

// ------------------------------------------------------------------------------------------------
// kernel dispatch helpers
// ------------------------------------------------------------------------------------------------
static void run_resid_norm(TSHipGpt* m, const char* name, int rows, ResidNormArgs a) {
    const int h = m->c.hidden;
#define TSHIP_RN(NPT)                                                                         \
    if (m->f16) launch(m, name, resid_norm_kernel<half_t, NPT>, dim3(rows), dim3(256), a);   \
    else launch(m, name, resid_norm_kernel<float, NPT>, dim3(rows), dim3(256), a);
    if (h <= 1024) { TSHIP_RN(4) } else if (h <= 2048) { TSHIP_RN(8) } else if (h <= 4096) { TSHIP_RN(16) } else { TSHIP_RN(32) }
#undef TSHIP_RN
}

// Y = X * W for <= 128 rows.  fp16: MFMA kernel; epilogue per `epi`.  fp32: tiled GEMM into partials.
static void run_skinny(TSHipGpt* m, const char* name, const GemmW& w, const void* X, long ldx, int rows, int epi, SkinnyArgs e) {
    TSHIP_REQUIRE(m->f16, "internal: run_skinny is the fp16 path");
    e.W = w.buf.as<half_t>(); e.KT = w.KT; e.NT = w.NT; e.X = (const half_t*)X; e.ldx = (int)ldx;
    e.KS = (epi == EPI_PARTIAL || epi == EPI_SPLIT_TAIL) ? w.KS : 1; e.rows_valid = rows;
    if (epi == EPI_SPLIT_TAIL) {
        // the exchange area holds [split][tile][1024] floats and one counter per tile
        TSHIP_REQUIRE(e.out == m->part_h.as<float>() && (size_t)e.KS * w.NT * 1024 * sizeof(float) <= m->part_h.bytes,
                      "internal: split-K exchange area too small");
        TSHIP_REQUIRE(e.tile_count == m->tile_count.as<int>() && (size_t)w.NT * sizeof(int) <= m->tile_count.bytes,
                      "internal: too few tile counters");
    }
    TSHIP_REQUIRE(epi != EPI_SPLIT_TAIL || (m->BT == 1 && e.tile_count), "internal: the split tail needs one batch tile and the tile counters");
    dim3 grid(w.NT * e.KS);
    const int BT = m->BT;
    if (epi == EPI_ACT16 && BT == 1) {
        // Column tiles per block.  A launch lasts as long as its busiest compute unit, and a unit's time goes with the
        // bytes it requests: the block's weight tiles and one copy of the activations (as large as one tile).  Costs in
        // half tiles: rounds of blocks over the units x (2 per tile + 2); 15 stands for a tile and a half per block.
        const int ncu = n_compute_units();
        int best = 10; long best_cost = ceil_div(w.NT, ncu) * 4;
        const long hb = 2 * (w.NT / 3) + w.NT % 3, hcost = ceil_div(hb, ncu) * 5;
        if (hcost < best_cost) { best = 15; best_cost = hcost; }
        for (int nj = 2; nj <= 4; ++nj) {
            const long cost = ceil_div(ceil_div(w.NT, nj), ncu) * (2 * nj + 2);
            if (cost < best_cost) { best = 10 * nj; best_cost = cost; }
        }
        if (g_hooks.ffn_tiles) best = g_hooks.ffn_tiles;
        if (best == 15) { launch_skinny(m, name, skinny_gemm_f16_kernel<1, EPI_ACT16, 8, 8, 2, true>, dim3((unsigned)hb), dim3(512), e); return; }
        if (best == 20) { launch_skinny(m, name, skinny_gemm_f16_kernel<1, EPI_ACT16, 8, 8, 2>, dim3((unsigned)ceil_div(w.NT, 2)), dim3(512), e); return; }
        if (best == 30) { launch_skinny(m, name, skinny_gemm_f16_kernel<1, EPI_ACT16, 8, 4, 3>, dim3((unsigned)ceil_div(w.NT, 3)), dim3(512), e); return; }
        if (best == 40) { launch_skinny(m, name, skinny_gemm_f16_kernel<1, EPI_ACT16, 8, 4, 4>, dim3((unsigned)ceil_div(w.NT, 4)), dim3(512), e); return; }
        TSHIP_REQUIRE(best == 10, "internal: column tiles per block");
    }
    TSHIP_REQUIRE(!e.Wtab, "internal: batched problems go through the kernel's BATCHED instantiations");
    if (BT == 1 && (epi == EPI_PARTIAL || epi == EPI_SPLIT_TAIL)) {
        // the first batch of a wavefront is requested whole (fragments beyond its k range are clamped duplicates): a batch as
        // long as the range keeps the requested bytes at the needed ones
        const long pw = ceil_div(ceil_div(w.KT, e.KS), 8);
        if (pw <= 2) {
            if (epi == EPI_PARTIAL) launch_skinny(m, name, skinny_gemm_f16_kernel<1, EPI_PARTIAL, 8, 2>, grid, dim3(512), e);
            else launch_skinny(m, name, skinny_gemm_f16_kernel<1, EPI_SPLIT_TAIL, 8, 2>, grid, dim3(512), e);
            return;
        }
        if (pw <= 4) {
            if (epi == EPI_PARTIAL) launch_skinny(m, name, skinny_gemm_f16_kernel<1, EPI_PARTIAL, 8, 4>, grid, dim3(512), e);
            else launch_skinny(m, name, skinny_gemm_f16_kernel<1, EPI_SPLIT_TAIL, 8, 4>, grid, dim3(512), e);
            return;
        }
    }
#define TSHIP_SK(BTV, NWV)                                                                                                  \
    if (epi == EPI_PARTIAL) launch_skinny(m, name, skinny_gemm_f16_kernel<BTV, EPI_PARTIAL, NWV>, grid, dim3(NWV * 64), e);        \
    else if (epi == EPI_F32_BIAS) launch_skinny(m, name, skinny_gemm_f16_kernel<BTV, EPI_F32_BIAS, NWV>, grid, dim3(NWV * 64), e); \
    else if (epi == EPI_RESID_TAIL) launch_skinny(m, name, skinny_gemm_f16_kernel<BTV, EPI_RESID_TAIL, NWV, (BTV == 1 ? 16 : 8)>, grid, dim3(NWV * 64), e); \
    else if (epi == EPI_SPLIT_TAIL) launch_skinny(m, name, skinny_gemm_f16_kernel<BTV, EPI_SPLIT_TAIL, NWV>, grid, dim3(NWV * 64), e); \
    else launch_skinny(m, name, skinny_gemm_f16_kernel<BTV, EPI_ACT16, NWV>, grid, dim3(NWV * 64), e);
    if (BT == 1) { TSHIP_SK(1, 8) } else if (BT == 2) { TSHIP_SK(2, 8) } else { TSHIP_SK(4, 4) }
#undef TSHIP_SK
}

static void run_gemm_f32(TSHipGpt* m, const char* name, const GemmW& w, const float* X, long ldx, int rows, float* out, long ld_out,
                         long split_stride, int KS, const float* bias = nullptr) {
    F32GemmArgs g;
    g.bias = KS == 1 ? bias : nullptr;
    g.A = X; g.lda = ldx; g.B = w.buf.as<float>(); g.ldb = w.ld; g.C = out; g.ldc = ld_out; g.split_stride = split_stride;
    g.M = rows; g.N = w.N; g.K = w.K; g.KS = KS;
    if (rows <= 32) {      // decode steps: every weight element once, up to 32 rows in registers
        dim3 sgrid((unsigned)ceil_div(w.N, 64), 1, KS);
        if (rows <= 8) launch(m, name, skinny_gemm_f32_kernel<8>, sgrid, dim3(256), g);
        else if (rows <= 16) launch(m, name, skinny_gemm_f32_kernel<16>, sgrid, dim3(256), g);
        else launch(m, name, skinny_gemm_f32_kernel<32>, sgrid, dim3(256), g);
        return;
    }
    dim3 grid((unsigned)ceil_div(w.N, 64), (unsigned)ceil_div(rows, 64), KS);
    launch(m, name, gemm_f32_kernel, grid, dim3(256), g);
}

// Y = X * W for many rows (prefill), fp16: LDS-tiled MFMA kernels from 512 rows on, 128 x 128 tiles below.  X row-major
// with at least round_up(R, 128) rows allocated (the small-tile kernel reads whole row tiles; rows from R on are never stored).
// n_problems > 1 (LDS-tiled asynchronous kernel only, see big_gemm_batched_ok): e.Wtab / rows_tab / strides describe that many
// problems of the same shape and at most R rows each, run by one launch.
static bool big_gemm_batched_ok(const GemmW& w, long R) { return R >= 512 && w.KT % 2 == 0; }
static void run_big_gemm(TSHipGpt* m, const char* name, const GemmW& w, const void* X, long ldx, long R, int epi, BigArgs e, int n_problems = 1) {
    const long Rp = round_up(R, 128);
    e.W = w.buf.as<half_t>(); e.KT = w.KT; e.NT = w.NT; e.X = (const half_t*)X; e.ldx = (int)ldx; e.R = (int)R;
    TSHIP_REQUIRE(n_problems == 1 || big_gemm_batched_ok(w, R), "internal: batched launch of a GEMM shape the LDS-tiled kernel does not take");
    if (R >= 512) {       // LDS-tiled kernel, 256 x 256 block tile
        constexpr int CK = 4;
        const unsigned shm = 2u * 2u * 8u * CK * 1024u;
        // one-dimensional grid of 8-row x 4-column tile patches, 32 blocks each, rounded up to whole rounds of 8 patches
        const long CT = ceil_div(w.NT, 8), RT = ceil_div(R, 256);
        long patches = ceil_div(CT, 4) * ceil_div(RT, 8);
        dim3 grid((unsigned)(round_up(patches, 8) * 32));
        if (w.KT % 2 == 0 && n_problems == 1) {
            // fewer than eight patches would leave XCDs without work: flatter patches (4, 2 or 1 row tiles)
            int ph = 8;
            while (ph > 1 && ceil_div(CT, 4) * ceil_div(RT, ph) < 8) ph /= 2;
            if (g_hooks.patch_rows) ph = g_hooks.patch_rows;
            patches = ceil_div(CT, 4) * ceil_div(RT, ph);
            e.patch_rows = ph;
            grid.x = (unsigned)(round_up(patches, 8) * 4 * ph);
        }
        if (n_problems > 1 && !e.packed_problems) { e.blocks_per_problem = (int)grid.x; grid.x *= (unsigned)n_problems; }
        if (w.KT % 2 == 0) {      // asynchronous staging: four stages of two k-tiles, eight wavefronts
            if (epi == BEPI_F32_BIAS) launch_shm(m, name, big_gemm3_f16_kernel<BEPI_F32_BIAS>, grid, dim3(512), shm, e);
            else if (epi == BEPI_RESID) launch_shm(m, name, big_gemm3_f16_kernel<BEPI_RESID>, grid, dim3(512), shm, e);
            else launch_shm(m, name, big_gemm3_f16_kernel<BEPI_ACT16>, grid, dim3(512), shm, e);
            return;
        }
        if (epi == BEPI_F32_BIAS) launch_shm(m, name, big_gemm2_f16_kernel<BEPI_F32_BIAS, CK>, grid, dim3(256), shm, e);
        else if (epi == BEPI_RESID) launch_shm(m, name, big_gemm2_f16_kernel<BEPI_RESID, CK>, grid, dim3(256), shm, e);
        else launch_shm(m, name, big_gemm2_f16_kernel<BEPI_ACT16, CK>, grid, dim3(256), shm, e);
        return;
    }
    dim3 grid((unsigned)ceil_div(w.NT, 4), (unsigned)(Rp / 128));
    if (epi == BEPI_F32_BIAS) launch(m, name, big_gemm_f16_kernel<BEPI_F32_BIAS>, grid, dim3(256), e);
    else if (epi == BEPI_RESID) launch(m, name, big_gemm_f16_kernel<BEPI_RESID>, grid, dim3(256), e);
    else launch(m, name, big_gemm_f16_kernel<BEPI_ACT16>, grid, dim3(256), e);
}

typedef void (*AttnKernel)(AttnArgs);
template <typename CT, typename AT, int D>
static AttnKernel pick_attn_g(int G, bool prefill) {
    switch (G) {
        case 1: return prefill ? attn_prefill_kernel<CT, AT, D, 1> : attn_decode_kernel<CT, AT, D, 1>;
        case 2: return prefill ? attn_prefill_kernel<CT, AT, D, 2> : attn_decode_kernel<CT, AT, D, 2>;
        case 4: return prefill ? attn_prefill_kernel<CT, AT, D, 4> : attn_decode_kernel<CT, AT, D, 4>;
        case 8: return prefill ? attn_prefill_kernel<CT, AT, D, 8> : attn_decode_kernel<CT, AT, D, 8>;
        case 3: return prefill ? attn_prefill_kernel<CT, AT, D, 3> : attn_decode_kernel<CT, AT, D, 3>;
        case 5: return prefill ? attn_prefill_kernel<CT, AT, D, 5> : attn_decode_kernel<CT, AT, D, 5>;
        case 6: return prefill ? attn_prefill_kernel<CT, AT, D, 6> : attn_decode_kernel<CT, AT, D, 6>;
        case 7: return prefill ? attn_prefill_kernel<CT, AT, D, 7> : attn_decode_kernel<CT, AT, D, 7>;
        default: throw Error("query heads per KV head must be 1 to 8");
    }
}
template <typename CT, typename AT>
static AttnKernel pick_attn_d(int D, int G, bool prefill) {
    switch (D) {
        case 16: return pick_attn_g<CT, AT, 16>(G, prefill);
        case 32: return pick_attn_g<CT, AT, 32>(G, prefill);
        case 64: return pick_attn_g<CT, AT, 64>(G, prefill);
        case 128: return pick_attn_g<CT, AT, 128>(G, prefill);
        default: throw Error("head_dim must be 16, 32, 64 or 128");
    }
}
template <int D>
static AttnKernel pick_attn_mfma(int G, bool prefill, bool split, bool ragged, int nq = 1) {
    if (prefill && nq == 2) {
        if (ragged) {
            switch (G) {
                case 1: return attn_mfma_prefill_kernel<D, 1, true, 2>;
                case 2: return attn_mfma_prefill_kernel<D, 2, true, 2>;
                case 4: return attn_mfma_prefill_kernel<D, 4, true, 2>;
                case 8: return attn_mfma_prefill_kernel<D, 8, true, 2>;
                default: throw Error("internal: two column groups per wavefront are for 1, 2, 4 or 8 query heads per KV head");
            }
        }
        switch (G) {
            case 1: return attn_mfma_prefill_kernel<D, 1, false, 2>;
            case 2: return attn_mfma_prefill_kernel<D, 2, false, 2>;
            case 4: return attn_mfma_prefill_kernel<D, 4, false, 2>;
            case 8: return attn_mfma_prefill_kernel<D, 8, false, 2>;
            default: throw Error("internal: two column groups per wavefront are for 1, 2, 4 or 8 query heads per KV head");
        }
    }
    if (prefill && ragged) {
        switch (G) {
            case 1: return attn_mfma_prefill_kernel<D, 1, true>;
            case 2: return attn_mfma_prefill_kernel<D, 2, true>;
            case 4: return attn_mfma_prefill_kernel<D, 4, true>;
            case 8: return attn_mfma_prefill_kernel<D, 8, true>;
            case 3: return attn_mfma_prefill_kernel<D, 3, true>;
            case 5: return attn_mfma_prefill_kernel<D, 5, true>;
            case 6: return attn_mfma_prefill_kernel<D, 6, true>;
            case 7: return attn_mfma_prefill_kernel<D, 7, true>;
            default: throw Error("query heads per KV head must be 1 to 8");
        }
    }
    TSHIP_REQUIRE(prefill, "internal: the MFMA decode kernels are picked by pick_attn_mfma_decode");
    (void)split;
    switch (G) {
        case 1: return attn_mfma_prefill_kernel<D, 1>;
        case 2: return attn_mfma_prefill_kernel<D, 2>;
        case 4: return attn_mfma_prefill_kernel<D, 4>;
        case 8: return attn_mfma_prefill_kernel<D, 8>;
        case 3: return attn_mfma_prefill_kernel<D, 3>;
        case 5: return attn_mfma_prefill_kernel<D, 5>;
        case 6: return attn_mfma_prefill_kernel<D, 6>;
        case 7: return attn_mfma_prefill_kernel<D, 7>;
        default: throw Error("query heads per KV head must be 1 to 8");
    }
}
// MFMA decode attention: leading scalar arguments (preloaded at wavefront start) in front of the struct
typedef void (*AttnDecodeKernel)(void*, int, int, int, int, int, int, int, int, unsigned, int, int, unsigned, AttnArgs);
// the decode kernel's leading arguments: one base pointer and 256-byte offsets from it (see AttnPacked)
static AttnPacked attn_pack_args(const AttnArgs& a) {
    auto off = [&](const void* p, const char* what) {
        if (!p) return 0;
        const long d = (const char*)p - (const char*)a.kcache;
        TSHIP_REQUIRE((d & 255) == 0 && (d >> 8) >= INT32_MIN && (d >> 8) <= INT32_MAX, std::string("internal: attention operand not at a 256-byte offset in reach of the key cache: ") + what);
        return (int)(d >> 8);
    };
    TSHIP_REQUIRE(a.max_len < (1L << 31) && a.ldq < (1L << 31) && a.split_stride < (1L << 31), "internal: attention strides beyond 32 bits");
    TSHIP_REQUIRE(a.H < 256 && a.Hkv < 256 && a.KS < 256 && a.ssq_nt < 65536 && a.ssq_ld < 65536 && a.kv_sub >= 0 && a.kv_sub < 32,
                  "internal: attention counts beyond their packed fields");
    AttnPacked p;
    p.kcache = a.kcache; p.d_vcache = off(a.vcache, "values"); p.d_qkv = off(a.qkv, "projection"); p.d_pos = off(a.d_pos, "position");
    p.d_bias = off(a.bias, "bias"); p.d_ssq = off(a.ssq, "tile sums"); p.d_rope_cos = off(a.rope_cos, "cosines"); p.d_rope_sin = off(a.rope_sin, "sines");
    p.max_len = (int)a.max_len;
    p.counts = (unsigned)a.H | ((unsigned)a.Hkv << 8) | ((unsigned)a.KS << 16) | (a.ssq ? 1u << 24 : 0u) | (a.rope_cos ? 1u << 25 : 0u) | (a.ln ? 1u << 26 : 0u) |
               ((unsigned)a.kv_sub << 27);
    p.ldq = (int)a.ldq; p.split_stride = (int)a.split_stride; p.ssq_dims = (unsigned)a.ssq_nt | ((unsigned)a.ssq_ld << 16);
    return p;
}
template <int D, bool SUB>
static AttnDecodeKernel pick_attn_mfma_decode_s(int G, bool split) {
    switch (G) {
        case 1: return split ? attn_mfma_kernel<D, 1, true, SUB> : attn_mfma_kernel<D, 1, false, SUB>;
        case 2: return split ? attn_mfma_kernel<D, 2, true, SUB> : attn_mfma_kernel<D, 2, false, SUB>;
        case 4: return split ? attn_mfma_kernel<D, 4, true, SUB> : attn_mfma_kernel<D, 4, false, SUB>;
        case 8: return split ? attn_mfma_kernel<D, 8, true, SUB> : attn_mfma_kernel<D, 8, false, SUB>;
        case 3: return split ? attn_mfma_kernel<D, 3, true, SUB> : attn_mfma_kernel<D, 3, false, SUB>;
        case 5: return split ? attn_mfma_kernel<D, 5, true, SUB> : attn_mfma_kernel<D, 5, false, SUB>;
        case 6: return split ? attn_mfma_kernel<D, 6, true, SUB> : attn_mfma_kernel<D, 6, false, SUB>;
        case 7: return split ? attn_mfma_kernel<D, 7, true, SUB> : attn_mfma_kernel<D, 7, false, SUB>;
        default: throw Error("query heads per KV head must be 1 to 8");
    }
}
// sub: the query heads of a KV head come in several groups (more than eight per KV head)
template <int D>
static AttnDecodeKernel pick_attn_mfma_decode(int G, bool split, bool sub) {
    return sub ? pick_attn_mfma_decode_s<D, true>(G, split) : pick_attn_mfma_decode_s<D, false>(G, split);
}
static AttnKernel pick_attn(TSHipGpt* m, bool prefill, bool split = false, bool ragged = false, int nq = 1) {
    if (m->vt) return m->D == 64 ? pick_attn_mfma<64>(m->G, prefill, split, ragged, nq) : pick_attn_mfma<128>(m->G, prefill, split, ragged, nq);
    return m->f16 ? pick_attn_d<half_t, half_t>(m->D, m->G, prefill) : pick_attn_d<float, float>(m->D, m->G, prefill);
}
template <typename CT>
static AttnKernel pick_kvw_t(int D) {
    switch (D) {
        case 16: return kv_write_kernel<CT, 16>;
        case 32: return kv_write_kernel<CT, 32>;
        case 64: return kv_write_kernel<CT, 64>;
        case 128: return kv_write_kernel<CT, 128>;
        default: throw Error("head_dim must be 16, 32, 64 or 128");
    }
}
static AttnKernel pick_kvw(TSHipGpt* m) { return m->f16 ? pick_kvw_t<half_t>(m->D) : pick_kvw_t<float>(m->D); }

static AttnArgs attn_args(TSHipGpt* m, LayerW& L) {
    AttnArgs a; std::memset(&a, 0, sizeof(a));
    a.bias = L.bqkv.as<float>(); a.H = m->c.n_heads; a.Hkv = m->c.n_kv_heads; a.kv_sub = m->SG;
    a.kcache = L.kc.p; a.vcache = L.vc.p; a.max_len = m->ML; a.vt = m->vt ? 1 : 0;
    if (m->c.use_rope) { a.rope_cos = m->rope_cos.as<float>(); a.rope_sin = m->rope_sin.as<float>(); }
    a.d_pos = m->d_pos.as<int>();
    a.scale = 1.0f / (float)std::sqrt((double)m->D);   // GroupQueryAttention.cs:193
    return a;
}

// decode attention: one block per (row, KV head), or several when that leaves CUs idle (MFMA kernels only)
static int attn_splits(TSHipGpt* m, int B) {
    if (!m->vt) return 1;
    const int NW = m->D == 128 ? 4 : 8;
    const long pairs = (long)B * m->Hv;
    long S = n_compute_units() / std::max<long>(pairs, 1);                  // fill the CUs
    // Splitting pays when a wavefront still walks many chunks: at a context of 1 k the launch is bound by its fixed
    // costs and the exchange adds 0.7 us (measured: 16.8 vs 15.9 us at 4 rows); at 8 k it gains 2.5 %.
    S = std::min<long>(S, (m->ML / 32) / (NW * 8L));
    if (g_hooks.attn_splits) S = g_hooks.attn_splits;      // (testing: force the number of blocks per pair)
    return (int)std::max<long>(1, std::min<long>(S, TSHipGpt::MAX_ATTN_SPLITS));
}
static void launch_attn_decode(TSHipGpt* m, AttnArgs a, int B) {
    if (!m->vt) { launch(m, "attn_decode", pick_attn(m, false), dim3(m->Hv, B), dim3(1024), a); return; }
    const int S = attn_splits(m, B);
    const unsigned threads = m->D == 128 ? 256 : 512;
    dim3 grid(m->c.n_kv_heads, B, m->SG);       // (one block per pair: the groups of a KV head's query heads on z)
    if (S > 1) {
        grid = dim3(m->Hv, B);
        const long pairs = (long)B * m->Hv, per = (long)m->G * m->D + 2 * m->G;
        TSHIP_REQUIRE((size_t)(pairs * S * per) * sizeof(float) <= m->attn_xchg.bytes && (size_t)pairs * sizeof(int) <= m->attn_count.bytes,
                      "internal: attention exchange area too small");
        a.S = S; a.xchg = m->attn_xchg.as<float>(); a.xcount = m->attn_count.as<int>();
        grid.z = (unsigned)S;
    }
    AttnDecodeKernel k = m->D == 64 ? pick_attn_mfma_decode<64>(m->G, S > 1, m->SG > 1) : pick_attn_mfma_decode<128>(m->G, S > 1, m->SG > 1);
    const AttnPacked p = attn_pack_args(a);
    launch(m, "attn_decode", k, grid, dim3(threads), p.kcache, p.d_vcache, p.d_qkv, p.d_pos, p.d_bias, p.d_ssq, p.d_rope_cos, p.d_rope_sin, p.max_len, p.counts,
           p.ldq, p.split_stride, p.ssq_dims, a);
}

// ------------------------------------------------------------------------------------------------
// MoE feed-forward at decode (MoEFeedForward.Process, Seq2SeqSharp/Layers/MoEFeedForward.cs:76-181)
// ------------------------------------------------------------------------------------------------
static void run_moe_ffn(TSHipGpt* m, LayerW& L, int rows, const ResidNormArgs& pre, const ResidNormArgs* next);
static void run_moe_ffn_prefill(TSHipGpt* m, LayerW& L, int rows, const ResidNormArgs& pre, const int* last_rows, int n_last, const ResidNormArgs* next);
static void moe_alloc(TSHipGpt* m);
static void moe_get_routing(TSHipGpt* m, int layer, float* top_idx, float* top_val, float* probs);
static void sample_tokens(TSHipGpt* m, int mode, float top_p, float temperature, const float* host_uniforms, const float* dev_uniforms, int B, int* gen_out, const int* d_step, bool record,
                          bool embed_next = false);
// tokens `d_ids` [rows][Tq] enter the sequences at indices pos0 ..: remember where each token occurred last
static void record_history(TSHipGpt* m, const int* d_ids, int rows, int Tq, int pos0) {
    if (!m->last_pos.p) return;
    TSHIP_REQUIRE(rows <= m->c.max_batch && (size_t)rows * m->last_ld * sizeof(int) <= m->last_pos.bytes, "internal: token history table too small");
    launch(m, "history", history_kernel, dim3((unsigned)ceil_div((long)rows * Tq, 256)), dim3(256), d_ids, rows, Tq, (long)Tq, pos0, (const int*)nullptr,
           (int)m->c.vocab, m->last_pos.as<int>(), m->last_ld);
}


// ------------------------------------------------------------------------------------------------
// decode step, deferred-norm form (fp16 weights, RMSNorm, dense feed-forward): 5 launches per layer.
//   gemm_qkv   : X = half(gamma1 * x) packed -> split-K partials
//   attn_decode: (sum partials) * rinv + bias, RoPE, cache append, attention
//   gemm_wo    : tail adds partials + b0 + x -> x, half(gamma2 * x), tile sums of squares
//   gemm_ffn13 : act((X W1) * rinv + b1) * ((X W3) * rinv + b3) -> packed fp16
//   gemm_ffn2  : tail as gemm_wo, with the next layer's (or the final) gamma
// rinv = 1 / sqrt(mean(x^2) + eps) is rebuilt by every consumer from the tile sums, so no launch exists only to
// normalise (RMSNormalization.Norm, Seq2SeqSharp/Layers/RMSNormalization.cs:33-37, folded into its neighbours).
// ------------------------------------------------------------------------------------------------
// first kernel of a decode step on the fused-norm path: embedding row x sqrt(h), the first layer's normalisation input, sums of squares
static FnPrepArgs embed_prepare_args(TSHipGpt* m, const int* d_ids) {
    const int h = m->c.hidden;
    FnPrepArgs a; std::memset(&a, 0, sizeof(a));
    a.x = m->x.as<float>(); a.ldx = h; a.h = h; a.ids = d_ids; a.emb = m->emb.p; a.emb_f16 = 1; a.emb_scale = (float)std::sqrt((double)h);
    a.seg = m->seg.as<float>();      // (a cached decode step feeds one token per sequence: segment 0, Decoder.cs:661-673)
    a.gamma = m->L[0]->n1_g.as<float>(); a.xg16 = m->xn.as<half_t>(); a.xg_kt = (int)(m->ldh / 16); a.ssq_out = m->ssq.as<float>(); a.ssq_ld = m->Bpad;
    a.ln = m->ln ? 1 : 0;
    return a;
}
static void decode_step_fn(TSHipGpt* m, const int* d_ids, int B) {
    auto& c = m->c;
    const int h = c.hidden, F = c.ffn_dim;
    const long hp = round_up(h, 32), qp = round_up(m->Nqkv, 32), Vp = round_up(c.vocab, 32);
    const int NTh = (int)(hp / 32), xkt = (int)(m->ldh / 16);
    float* ssq = m->ssq.as<float>();
    auto with_ssq = [&](SkinnyArgs& e) { e.ssq = ssq; e.ssq_nt = NTh; e.ssq_ld = m->Bpad; e.inv_h = 1.0f / (float)h; e.eps = c.norm_eps; e.ln = m->ln ? 1 : 0; };
    auto tail = [&](SkinnyArgs& e, const float* bias, const float* gamma) {
        e.out = m->part_h.as<float>(); e.ld_out = (int)hp; e.split_stride = (long)m->Bpad * hp;
        e.bias = bias; e.n_valid = h; e.x = m->x.as<float>(); e.ldx_res = h; e.gamma = gamma;
        e.xg16 = m->xn.as<half_t>(); e.xg_kt = xkt; e.ssq_out = ssq; e.ssq_out_ld = m->Bpad;
        e.ln = m->ln ? 1 : 0;      // (LayerNorm: the tails also store the tiles' plain sums)
    };
    if (m->embed_done) {
        m->embed_done = false;        // (the greedy sampling kernel went on to embed the tokens it chose)
    } else {
        FnPrepArgs a = embed_prepare_args(m, d_ids);
        if (h <= 2048) launch(m, "embed_prepare", fn_prepare_kernel<8>, dim3(B), dim3(256), a);
        else if (h <= 4096) launch(m, "embed_prepare", fn_prepare_kernel<16>, dim3(B), dim3(256), a);
        else launch(m, "embed_prepare", fn_prepare_kernel<32>, dim3(B), dim3(256), a);
    }
    for (int l = 0; l < c.n_layers; ++l) {
        LayerW& L = *m->L[l];
        const long qstride = (long)m->Bpad * qp;
        {
            SkinnyArgs e; std::memset(&e, 0, sizeof(e));
            e.out = m->part_qkv.as<float>(); e.ld_out = (int)qp; e.split_stride = qstride;
            run_skinny(m, "gemm_qkv", L.qkv, m->xn.p, m->ldh, B, EPI_PARTIAL, e);
        }
        {
            AttnArgs a = attn_args(m, L);
            a.qkv = m->part_qkv.as<float>(); a.KS = L.qkv.KS; a.split_stride = qstride; a.ldq = qp;
            a.out = m->o.p; a.ld_out = m->ldh; a.out_kt = xkt;
            a.ssq = ssq; a.ssq_nt = NTh; a.ssq_ld = m->Bpad; a.inv_h = 1.0f / (float)h; a.eps = c.norm_eps;
            if (m->ln) { a.ln = 1; a.bias = L.ln_qkv.as<float>(); TSHIP_REQUIRE(a.ldq == qp, "internal: folded LayerNorm constants are laid out by the projection's leading dimension"); }
            launch_attn_decode(m, a, B);
        }
        {
            SkinnyArgs e; std::memset(&e, 0, sizeof(e));
            tail(e, L.bo.as<float>(), L.n2_g.as<float>());
            if (L.wo.KS > 1) {
                e.out = m->part_h.as<float>(); e.tile_count = m->tile_count.as<int>();
                run_skinny(m, "gemm_wo", L.wo, m->o.p, m->ldh, B, EPI_SPLIT_TAIL, e);
            } else {
                run_skinny(m, "gemm_wo", L.wo, m->o.p, m->ldh, B, EPI_RESID_TAIL, e);
            }
        }
        {
            SkinnyArgs e; std::memset(&e, 0, sizeof(e));
            e.bias = L.b1.as<float>(); e.bias2 = L.b3.as<float>(); e.out16 = m->a.as<half_t>(); e.ld16 = (int)m->ldF;
            e.act = c.act; e.gated = m->gated; e.n_valid = F; e.out16_kt = L.w2.KT;
            with_ssq(e);
            if (m->ln) { e.ln_d = L.ln_13.as<float>(); e.ln_c = L.ln_13.as<float>() + (long)L.w13.NT * 32; }
            run_skinny(m, "gemm_ffn13", L.w13, m->xn.p, m->ldh, B, EPI_ACT16, e);
        }
        const float* next_gamma = l + 1 < c.n_layers ? m->L[l + 1]->n1_g.as<float>() : m->fn_g.as<float>();
        if (L.w2.KS == 1) {
            SkinnyArgs e; std::memset(&e, 0, sizeof(e));
            tail(e, L.b2.as<float>(), next_gamma);
            run_skinny(m, "gemm_ffn2", L.w2, m->a.p, m->ldF, B, EPI_RESID_TAIL, e);
        } else if (m->BT == 1) {
            // long K: split across blocks so that every CU streams weights; the block of a column tile that finishes
            // last adds the partial sums and performs the tail
            SkinnyArgs e; std::memset(&e, 0, sizeof(e));
            tail(e, L.b2.as<float>(), next_gamma);
            e.out = m->part_h.as<float>();       // exchange area [split][tile][1024]: 16 * Bpad * hp floats hold it for Bpad = 32
            e.tile_count = m->tile_count.as<int>();
            run_skinny(m, "gemm_ffn2", L.w2, m->a.p, m->ldF, B, EPI_SPLIT_TAIL, e);
        } else {
            // long K: split across blocks so that every CU streams weights, then a small tail kernel
            SkinnyArgs e; std::memset(&e, 0, sizeof(e));
            e.out = m->part_h.as<float>(); e.ld_out = (int)hp; e.split_stride = (long)m->Bpad * hp;
            run_skinny(m, "gemm_ffn2", L.w2, m->a.p, m->ldF, B, EPI_PARTIAL, e);
            ResidTailArgs r; std::memset(&r, 0, sizeof(r));
            r.x = m->x.as<float>(); r.ldx = h; r.h = h; r.rows = B;
            r.part = m->part_h.as<float>(); r.KS = L.w2.KS; r.split_stride = (long)m->Bpad * hp; r.ld_part = hp; r.bias = L.b2.as<float>();
            r.gamma = next_gamma; r.xg16 = m->xn.as<half_t>(); r.xg_kt = xkt; r.ssq_out = ssq; r.ssq_ld = m->Bpad;
            if (m->BT == 1) launch(m, "resid_tail", resid_tail_kernel<4>, dim3(NTh), dim3(256), r);
            else if (m->BT == 2) launch(m, "resid_tail", resid_tail_kernel<8>, dim3(NTh), dim3(256), r);
            else launch(m, "resid_tail", resid_tail_kernel<16>, dim3(NTh), dim3(256), r);
        }
    }
    {
        SkinnyArgs e; std::memset(&e, 0, sizeof(e));
        e.out = m->logits.as<float>(); e.ld_out = (int)Vp; e.bias = m->head_b.as<float>(); e.n_valid = c.vocab;
        with_ssq(e);
        if (m->ln) { e.ln_d = m->ln_head.as<float>(); e.ln_c = m->ln_head.as<float>() + Vp; }
        e.advance_pos = m->d_pos.as<int>();
        run_skinny(m, "gemm_head", m->head, m->xn.p, m->ldh, B, EPI_F32_BIAS, e);
    }
    m->pos += 1;
}

// ------------------------------------------------------------------------------------------------
// decode step: tokens (device int32 [batch]) -> logits (device fp32 [batch][vocab])
// ------------------------------------------------------------------------------------------------
static void decode_step(TSHipGpt* m, const int* d_ids, int B) {
    if (m->fused_norm) { decode_step_fn(m, d_ids, B); return; }
    auto& c = m->c;
    const int h = c.hidden, F = c.ffn_dim;
    const long hp = round_up(h, 32), qp = round_up(m->Nqkv, 32);
    ResidNormArgs rn; std::memset(&rn, 0, sizeof(rn));
    rn.x = m->x.as<float>(); rn.ldx = h; rn.h = h; rn.eps = c.norm_eps; rn.norm_type = c.norm_type;
    rn.xn = m->xn.p; rn.ldxn = m->ldh; rn.xn_kt = m->f16 ? (int)(m->ldh / 16) : 0;

    // embedding gather * sqrt(h) and the first layer's attention norm
    {
        ResidNormArgs a = rn;
        a.ids = d_ids; a.emb = m->emb.p; a.emb_f16 = m->f16; a.emb_scale = (float)std::sqrt((double)h);
        a.seg = m->seg.as<float>();      // (a cached decode step feeds one token per sequence: segment 0, Decoder.cs:661-673)
        a.gamma = m->L[0]->n1_g.as<float>(); a.beta = m->L[0]->n1_b.as<float>();
        run_resid_norm(m, "embed_norm", B, a);
    }
    for (int l = 0; l < c.n_layers; ++l) {
        LayerW& L = *m->L[l];
        // QKV projection -> split-K partials
        long qstride = (long)m->Bpad * qp;
        if (m->f16) {
            SkinnyArgs e; std::memset(&e, 0, sizeof(e));
            e.out = m->part_qkv.as<float>(); e.ld_out = (int)qp; e.split_stride = qstride;
            run_skinny(m, "gemm_qkv", L.qkv, m->xn.p, m->ldh, B, EPI_PARTIAL, e);
        } else {
            run_gemm_f32(m, "gemm_qkv", L.qkv, m->xn.as<float>(), m->ldh, B, m->part_qkv.as<float>(), qp, qstride, L.qkv.KS);
        }
        // RoPE, cache append, attention
        {
            AttnArgs a = attn_args(m, L);
            a.qkv = m->part_qkv.as<float>(); a.KS = L.qkv.KS; a.split_stride = qstride; a.ldq = qp;
            a.out = m->o.p; a.ld_out = m->ldh; a.out_kt = m->f16 ? (int)(m->ldh / 16) : 0;
            launch_attn_decode(m, a, B);
        }
        // output projection -> partials
        long hstride = (long)m->Bpad * hp;
        if (m->f16) {
            SkinnyArgs e; std::memset(&e, 0, sizeof(e));
            e.out = m->part_h.as<float>(); e.ld_out = (int)hp; e.split_stride = hstride;
            run_skinny(m, "gemm_wo", L.wo, m->o.p, m->ldh, B, EPI_PARTIAL, e);
        } else {
            run_gemm_f32(m, "gemm_wo", L.wo, m->o.as<float>(), m->ldh, B, m->part_h.as<float>(), hp, hstride, L.wo.KS);
        }
        // x += attn_out + b0 ; feed-forward norm
        ResidNormArgs a2 = rn;
        a2.part = m->part_h.as<float>(); a2.KS = L.wo.KS; a2.split_stride = hstride; a2.ld_part = hp; a2.bias = L.bo.as<float>();
        a2.gamma = L.n2_g.as<float>(); a2.beta = L.n2_b.as<float>();
        const float* next_g = (l + 1 < c.n_layers) ? m->L[l + 1]->n1_g.as<float>() : m->fn_g.as<float>();
        const float* next_b = (l + 1 < c.n_layers) ? m->L[l + 1]->n1_b.as<float>() : m->fn_b.as<float>();
        if (L.moe) {
            a2.norm_type = 1;          // MoEFeedForward always uses LayerNormalization (MoEFeedForward.cs:49)
            // the next norm's kernel adds the experts' outputs to x first
            ResidNormArgs a3 = rn;
            a3.gamma = next_g; a3.beta = next_b;
            if (l + 1 == c.n_layers) a3.advance_pos = m->d_pos.as<int>();
            run_moe_ffn(m, L, B, a2, &a3);
            continue;
        }
        run_resid_norm(m, "resid_norm_ffn", B, a2);
        // FFN up (and gate) projection
        if (m->f16) {
            SkinnyArgs e; std::memset(&e, 0, sizeof(e));
            e.bias = L.b1.as<float>(); e.bias2 = L.b3.as<float>(); e.out16 = m->a.as<half_t>(); e.ld16 = (int)m->ldF;
            e.act = c.act; e.gated = m->gated; e.n_valid = F; e.out16_kt = L.w2.KT;
            run_skinny(m, "gemm_ffn13", L.w13, m->xn.p, m->ldh, B, EPI_ACT16, e);
        } else {
            long fp = m->F13, fstride = (long)m->Bpad * fp;
            run_gemm_f32(m, "gemm_ffn13", L.w13, m->xn.as<float>(), m->ldh, B, m->part_f.as<float>(), fp, fstride, L.w13.KS);
            long tot = (long)B * F;
            launch(m, "ffn_act", ffn_act_kernel<float>, dim3((unsigned)ceil_div(tot, 256)), dim3(256), (const float*)m->part_f.as<float>(), L.w13.KS,
                   fstride, fp, (const float*)L.b1.as<float>(), (const float*)L.b3.as<float>(), F, (int)m->gated, (int)c.act, m->a.as<float>(), m->ldF, (long)B);
        }
        // FFN down projection -> partials
        if (m->f16) {
            SkinnyArgs e; std::memset(&e, 0, sizeof(e));
            e.out = m->part_h.as<float>(); e.ld_out = (int)hp; e.split_stride = hstride;
            run_skinny(m, "gemm_ffn2", L.w2, m->a.p, m->ldF, B, EPI_PARTIAL, e);
        } else {
            run_gemm_f32(m, "gemm_ffn2", L.w2, m->a.as<float>(), m->ldF, B, m->part_h.as<float>(), hp, hstride, L.w2.KS);
        }
        // x += ffn_out + b2 ; next layer's attention norm, or the final norm
        ResidNormArgs a3 = rn;
        a3.part = m->part_h.as<float>(); a3.KS = L.w2.KS; a3.split_stride = hstride; a3.ld_part = hp; a3.bias = L.b2.as<float>();
        a3.gamma = next_g; a3.beta = next_b;
        if (l + 1 == c.n_layers) a3.advance_pos = m->d_pos.as<int>();
        run_resid_norm(m, l + 1 == c.n_layers ? "resid_norm_final" : "resid_norm_attn", B, a3);
    }
    // vocabulary projection (only the new position exists at decode)
    const long Vp = round_up(c.vocab, 32);
    if (m->f16) {
        SkinnyArgs e; std::memset(&e, 0, sizeof(e));
        e.out = m->logits.as<float>(); e.ld_out = (int)Vp; e.bias = m->head_b.as<float>(); e.n_valid = c.vocab;
        run_skinny(m, "gemm_head", m->head, m->xn.p, m->ldh, B, EPI_F32_BIAS, e);
    } else {
        run_gemm_f32(m, "gemm_head", m->head, m->xn.as<float>(), m->ldh, B, m->logits.as<float>(), Vp, 0, 1, m->head_b.as<float>());
    }
    m->pos += 1;
}

// ------------------------------------------------------------------------------------------------
// prefill: whole prompts, causal attention, cache filled for every position, logits of the last position
// ------------------------------------------------------------------------------------------------
// host_lens (optional): the sequences were padded to Tp tokens; their original lengths select BuildSelfTriMask's masking
static void prefill(TSHipGpt* m, const int32_t* host_ids, int B, int Tp, const int32_t* host_lens = nullptr) {
    auto& c = m->c;
    const int h = c.hidden, F = c.ffn_dim;
    const long R = (long)B * Tp, Rp = round_up(R, 128);
    const long qp = round_up(m->Nqkv, 32);
    const int pos0 = m->pos;              // tokens are appended behind what the cache holds (nothing after Create / Reset)
    TSHIP_REQUIRE(pos0 == 0 || m->cur_batch == B, "TSHip_GptPrefill: batch differs from the cached sequences; call TSHip_GptReset first");
    TSHIP_REQUIRE(Tp >= 1 && pos0 + Tp < c.max_seq_len, "TSHip_GptPrefill: prompt length exceeds max_seq_len");
    // prefill workspace: kept in the model and only ever grown, so that repeated prefills do not pay for allocation
    DevBuf &ids = m->pw_ids, &px = m->pw_x, &pxn = m->pw_xn, &pqkv = m->pw_qkv, &po = m->pw_o, &pa = m->pw_a, &pf = m->pw_f, &rowmap = m->pw_rowmap;
    ids.reserve(R * sizeof(int));
    TSHIP_CHECK_HIP(hipMemcpyAsync(ids.p, host_ids, R * sizeof(int), hipMemcpyHostToDevice, stream()));
    record_history(m, ids.as<int>(), B, Tp, pos0);
    if (m->seg.p) {
        // the segment of a token = the separators before it in this call's token list of its sequence (TensorUtils.cs:60-72)
        std::vector<int> sg((size_t)R);
        for (int b = 0; b < B; ++b) {
            int s_idx = 0;
            for (int j = 0; j < Tp; ++j) {
                TSHIP_REQUIRE(s_idx < c.max_segments, "TSHip_GptPrefill: a sequence holds more separator tokens than the model has segment embeddings");
                sg[(size_t)b * Tp + j] = s_idx;
                if (host_ids[(size_t)b * Tp + j] == c.sep_token_id) ++s_idx;
            }
        }
        m->pw_seg.reserve((size_t)R * sizeof(int));
        TSHIP_CHECK_HIP(hipMemcpyAsync(m->pw_seg.p, sg.data(), (size_t)R * sizeof(int), hipMemcpyHostToDevice, stream()));
        TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));       // (the host vector is a local)
    }
    std::vector<int> map(B);             // row of every sequence's last position
    for (int b = 0; b < B; ++b) map[b] = Tp * (b + 1) - 1;
    rowmap.reserve(B * sizeof(int));
    TSHIP_CHECK_HIP(hipMemcpyAsync(rowmap.p, map.data(), B * sizeof(int), hipMemcpyHostToDevice, stream()));
    if (host_lens) {
        TSHIP_REQUIRE(pos0 == 0, "TSHip_GptPrefillPadded: padded prompts start a sequence; call TSHip_GptReset first");
        m->pw_lens.reserve(B * sizeof(int));
        TSHIP_CHECK_HIP(hipMemcpyAsync(m->pw_lens.p, host_lens, B * sizeof(int), hipMemcpyHostToDevice, stream()));
    }
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));       // (map is a local; the copies must not outlive their sources)
    px.reserve((size_t)Rp * h * sizeof(float));
    pxn.reserve((size_t)Rp * m->ldh * m->esz());
    pqkv.reserve((size_t)Rp * qp * sizeof(float));
    po.reserve((size_t)Rp * m->ldh * m->esz());
    bool any_dense = false; for (auto& L : m->L) any_dense = any_dense || !L->moe;
    if (any_dense) pa.reserve((size_t)Rp * m->ldF * m->esz());
    if (!m->f16 && any_dense) pf.reserve((size_t)Rp * m->F13 * sizeof(float));

    ResidNormArgs rn; std::memset(&rn, 0, sizeof(rn));
    rn.x = px.as<float>(); rn.ldx = h; rn.h = h; rn.eps = c.norm_eps; rn.norm_type = c.norm_type;
    rn.xn = pxn.p; rn.ldxn = m->ldh;
    // Deferred RMSNorm (fp16 RMSNorm models, LDS-tiled GEMMs): no norm kernels.  The producer of the residual stream
    // stores half(gamma * x) and per-(32-column tile, row) sums of squares, a one-thread-per-row kernel turns those into
    // 1 / rms, and the consuming GEMMs scale their output rows by it.
    const bool deferred = m->fused_norm && !m->ln && R >= 512;
    const int NTh = (int)(round_up(h, 32) / 32);
    DevBuf &pssq = m->pw_ssq, &prinv = m->pw_rinv;
    auto make_rinv = [&](const char* name) {
        launch(m, name, rinv_rows_kernel, dim3((unsigned)ceil_div(R, 256)), dim3(256), (const float*)pssq.as<float>(), NTh, R, 1.0f / (float)h,
               c.norm_eps, prinv.as<float>(), R);
    };
    if (deferred) {
        pssq.reserve((size_t)NTh * R * sizeof(float));
        prinv.reserve((size_t)R * sizeof(float));
        FnPrepArgs a; std::memset(&a, 0, sizeof(a));
        a.x = px.as<float>(); a.ldx = h; a.h = h;
        a.ids = ids.as<int>(); a.emb = m->emb.p; a.emb_f16 = m->f16; a.emb_scale = (float)std::sqrt((double)h);
        a.seg = m->seg.as<float>(); a.seg_ids = m->seg.p ? m->pw_seg.as<int>() : nullptr;
        a.gamma = m->L[0]->n1_g.as<float>(); a.xg16 = pxn.as<half_t>(); a.xg_kt = 0; a.xg_ld = m->ldh; a.ssq_out = pssq.as<float>(); a.ssq_ld = R;
        if (h <= 2048) launch(m, "p_embed_prepare", fn_prepare_kernel<8>, dim3((unsigned)R), dim3(256), a);
        else if (h <= 4096) launch(m, "p_embed_prepare", fn_prepare_kernel<16>, dim3((unsigned)R), dim3(256), a);
        else launch(m, "p_embed_prepare", fn_prepare_kernel<32>, dim3((unsigned)R), dim3(256), a);
        make_rinv("p_rinv_attn");
    } else {
        ResidNormArgs a = rn;
        a.ids = ids.as<int>(); a.emb = m->emb.p; a.emb_f16 = m->f16; a.emb_scale = (float)std::sqrt((double)h);
        a.seg = m->seg.as<float>(); a.seg_ids = m->seg.p ? m->pw_seg.as<int>() : nullptr;
        a.gamma = m->L[0]->n1_g.as<float>(); a.beta = m->L[0]->n1_b.as<float>();
        run_resid_norm(m, "p_embed_norm", (int)R, a);
    }
    auto producer = [&](BigArgs& e, const float* gamma) {        // residual GEMM that also emits the next GEMM's input
        e.xg16 = pxn.as<half_t>(); e.ld_xg = (int)m->ldh; e.gamma = gamma; e.ssq_out = pssq.as<float>(); e.ssq_ld = R;
    };
    auto big = [&](const char* name, const GemmW& w, const void* X, long ldx, int epi, BigArgs e) { run_big_gemm(m, name, w, X, ldx, R, epi, e); };
    DevBuf& zero_bias = m->pw_zero_bias; zero_bias.reserve((size_t)std::max<long>(std::max<long>(qp, m->F13), round_up(h, 32)) * sizeof(float));
    for (int l = 0; l < c.n_layers; ++l) {
        LayerW& L = *m->L[l];
        AttnArgs aa = attn_args(m, L);
        aa.qkv = pqkv.as<float>(); aa.KS = 1; aa.split_stride = 0; aa.ldq = qp; aa.pos0 = pos0; aa.Tq = Tp;
        aa.out = po.p; aa.ld_out = m->ldh;
        aa.lens = host_lens ? m->pw_lens.as<int>() : nullptr;
        // The LDS-tiled QKV projection writes keys and values into the fragment-major cache itself (rotation included)
        // when its wavefronts' 64 x 128 tiles are whole chunks of whole heads; otherwise a kernel of its own does.
        const int HD = c.n_heads * m->D, GD = c.n_kv_heads * m->D;
        const bool fuse_kv = m->f16 && m->vt && pos0 % 32 == 0 && Tp % 32 == 0 && HD % 128 == 0 && GD % 128 == 0 && R >= 512 && L.qkv.KT % 2 == 0 &&
                             (m->D == 64 || m->D == 128) && !g_hooks.no_kv_fuse;
        if (m->f16) {
            BigArgs e; std::memset(&e, 0, sizeof(e));
            e.out = pqkv.as<float>(); e.ld_out = (int)qp; e.bias = L.bqkv.as<float>(); e.n_valid = m->Nqkv;
            if (deferred) e.rinv = prinv.as<float>();
            if (fuse_kv) {
                TSHIP_REQUIRE((long)round_up(pos0 + Tp, 32) <= m->ML, "internal: cache chunk beyond the allocation");
                e.kcache = (half_t*)L.kc.p; e.vcache = (half_t*)L.vc.p; e.kv_max_len = m->ML; e.kv_col0 = HD; e.kv_gd = GD; e.kv_D = m->D;
                e.kv_hkv = c.n_kv_heads; e.kv_Tq = Tp; e.kv_pos0 = pos0; e.rope_cos = aa.rope_cos; e.rope_sin = aa.rope_sin;
            }
            big("p_gemm_qkv", L.qkv, pxn.p, m->ldh, BEPI_F32_BIAS, e);
            aa.bias = zero_bias.as<float>();      // bias already added by the GEMM epilogue
        } else {
            run_gemm_f32(m, "p_gemm_qkv", L.qkv, pxn.as<float>(), m->ldh, (int)R, pqkv.as<float>(), qp, 0, 1);
        }
        if (fuse_kv) {
            // (cache written by the projection)
        } else if (m->vt && aa.pos0 % 32 == 0) {      // whole fragments, one block per 32-position chunk
            TSHIP_REQUIRE(qp % 4 == 0 && (long)round_up(aa.pos0 + Tp, 32) <= m->ML, "internal: cache chunk beyond the allocation");
            dim3 grid((unsigned)ceil_div(Tp, 32), c.n_kv_heads, B);
            if (m->D == 64) launch(m, "p_kv_write", kv_write_frag_kernel<64>, grid, dim3(256), aa);
            else launch(m, "p_kv_write", kv_write_frag_kernel<128>, grid, dim3(512), aa);
        } else {
            launch(m, "p_kv_write", pick_kvw(m), dim3(Tp, B), dim3(256), aa);
        }
        if (m->vt) {      // a wavefront per 16 / G query positions, 8 (head_dim 64) or 4 (head_dim 128) wavefronts per block
            // Two groups of 16 MFMA columns per wavefront (half the LDS fragment reads per score) at head size 128,
            // once the prompt is long enough for the coarser blocks to fill the chip.  (At head size 64 the second
            // group costs the second block per compute unit its registers and measured the same.)
            int nq = (m->D == 128 && 16 % m->G == 0 && (long)ceil_div(Tp, (16 / m->G) * 16) * m->Hv * B >= 2048) ? 2 : 1;
            if (g_hooks.attn_nq && 16 % m->G == 0) nq = g_hooks.attn_nq;
            const int per_block = (16 / m->G) * 8 * nq;
            launch(m, "p_attn", pick_attn(m, true, false, host_lens != nullptr, nq), dim3((unsigned)ceil_div(Tp, per_block), m->Hv, B), dim3(512), aa);
        }
        else launch(m, "p_attn", pick_attn(m, true), dim3(Tp, m->Hv, B), dim3(256), aa);
        ResidNormArgs a2 = rn;
        a2.gamma = L.n2_g.as<float>(); a2.beta = L.n2_b.as<float>();
        if (m->f16) {
            BigArgs e; std::memset(&e, 0, sizeof(e));
            e.out = px.as<float>(); e.ld_out = h; e.bias = L.bo.as<float>(); e.n_valid = h;
            if (deferred) producer(e, L.n2_g.as<float>());
            big("p_gemm_wo", L.wo, po.p, m->ldh, BEPI_RESID, e);
        } else {
            run_gemm_f32(m, "p_gemm_wo", L.wo, po.as<float>(), m->ldh, (int)R, pqkv.as<float>(), qp, 0, 1);
            a2.part = pqkv.as<float>(); a2.KS = 1; a2.ld_part = qp; a2.bias = L.bo.as<float>();
        }
        ResidNormArgs a3 = rn;
        if (l + 1 < c.n_layers) { a3.gamma = m->L[l + 1]->n1_g.as<float>(); a3.beta = m->L[l + 1]->n1_b.as<float>(); }
        else a3.xn = nullptr;
        const bool norm_after = !deferred && (l + 1 < c.n_layers || !m->f16);
        if (L.moe) {
            // the router kernel applies the pending attention output (fp32 models) and the layer's own LayerNorm; the
            // experts' output is added to the residual stream by the norm kernel that follows (a combine kernel of its own
            // behind the last layer of an fp16 model, which no norm kernel follows)
            run_moe_ffn_prefill(m, L, (int)R, a2, rowmap.as<int>(), B, norm_after ? &a3 : nullptr);
        } else if (deferred) make_rinv("p_rinv_ffn");
        else run_resid_norm(m, "p_norm_ffn", (int)R, a2);
        if (L.moe) {
            // (nothing more: no dense feed-forward in this layer)
        } else if (m->f16) {
            BigArgs e; std::memset(&e, 0, sizeof(e));
            e.bias = L.b1.as<float>(); e.bias2 = L.b3.as<float>(); e.out16 = pa.as<half_t>(); e.ld16 = (int)m->ldF;
            e.act = c.act; e.gated = m->gated; e.n_valid = F;
            if (deferred) e.rinv = prinv.as<float>();
            big("p_gemm_ffn13", L.w13, pxn.p, m->ldh, BEPI_ACT16, e);
            BigArgs e2; std::memset(&e2, 0, sizeof(e2));
            e2.out = px.as<float>(); e2.ld_out = h; e2.bias = L.b2.as<float>(); e2.n_valid = h;
            if (deferred && l + 1 < c.n_layers) producer(e2, m->L[l + 1]->n1_g.as<float>());
            big("p_gemm_ffn2", L.w2, pa.p, m->ldF, BEPI_RESID, e2);
        } else {
            run_gemm_f32(m, "p_gemm_ffn13", L.w13, pxn.as<float>(), m->ldh, (int)R, pf.as<float>(), m->F13, 0, 1);
            long tot = R * F;
            launch(m, "p_ffn_act", ffn_act_kernel<float>, dim3((unsigned)ceil_div(tot, 256)), dim3(256), (const float*)pf.as<float>(), 1, 0L,
                   (long)m->F13, (const float*)L.b1.as<float>(), (const float*)L.b3.as<float>(), F, (int)m->gated, (int)c.act, pa.as<float>(), m->ldF, R);
            run_gemm_f32(m, "p_gemm_ffn2", L.w2, pa.as<float>(), m->ldF, (int)R, pqkv.as<float>(), qp, 0, 1);
            a3.part = pqkv.as<float>(); a3.KS = 1; a3.ld_part = qp; a3.bias = L.b2.as<float>();
        }
        if (deferred) { if (l + 1 < c.n_layers) make_rinv("p_rinv_attn"); }
        else if (norm_after && !L.moe) run_resid_norm(m, "p_norm_attn", (int)R, a3);
    }
    // last position of every sequence (Decoder.cs:705-716) -> final norm -> vocabulary projection
    if (m->fused_norm && !m->ln) {
        FnPrepArgs a; std::memset(&a, 0, sizeof(a));
        a.x = m->x.as<float>(); a.ldx = h; a.h = h; a.src = px.as<float>(); a.ld_src = h; a.row_map = rowmap.as<int>();
        a.gamma = m->fn_g.as<float>(); a.xg16 = m->xn.as<half_t>(); a.xg_kt = (int)(m->ldh / 16); a.ssq_out = m->ssq.as<float>(); a.ssq_ld = m->Bpad;
        if (h <= 2048) launch(m, "p_final_prepare", fn_prepare_kernel<8>, dim3(B), dim3(256), a);
        else if (h <= 4096) launch(m, "p_final_prepare", fn_prepare_kernel<16>, dim3(B), dim3(256), a);
        else launch(m, "p_final_prepare", fn_prepare_kernel<32>, dim3(B), dim3(256), a);
    } else {
        ResidNormArgs a = rn;
        a.row_map = rowmap.as<int>(); a.xn = m->xn.p; a.ldxn = m->ldh; a.xn_kt = m->f16 ? (int)(m->ldh / 16) : 0;
        a.gamma = m->fn_g.as<float>(); a.beta = m->fn_b.as<float>();
        run_resid_norm(m, "p_final_norm", B, a);
    }
    const long Vp = round_up(c.vocab, 32);
    if (m->f16) {
        SkinnyArgs e; std::memset(&e, 0, sizeof(e));
        e.out = m->logits.as<float>(); e.ld_out = (int)Vp; e.bias = m->head_b.as<float>(); e.n_valid = c.vocab;
        if (m->fused_norm && !m->ln) { e.ssq = m->ssq.as<float>(); e.ssq_nt = (int)(round_up(h, 32) / 32); e.ssq_ld = m->Bpad; e.inv_h = 1.0f / (float)h; e.eps = c.norm_eps; }
        run_skinny(m, "gemm_head", m->head, m->xn.p, m->ldh, B, EPI_F32_BIAS, e);
    } else {
        run_gemm_f32(m, "gemm_head", m->head, m->xn.as<float>(), m->ldh, B, m->logits.as<float>(), Vp, 0, 1, m->head_b.as<float>());
    }
    m->pos = pos0 + Tp;
    TSHIP_CHECK_HIP(hipMemcpyAsync(m->d_pos.p, &m->pos, sizeof(int), hipMemcpyHostToDevice, stream()));
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    m->cur_batch = B;
}

}  // namespace tship

#include "tship_gpt_extra.h"
#include "tship_beam.h"

// =================================================================================================
// exported functions
// =================================================================================================
extern "C" {

TSHIP_API int TSHip_GptCreate(const TSHipGptConfig* cfg, TSHipGpt** out) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(cfg && out, "TSHip_GptCreate: null argument");
    ensure_init();
    const TSHipGptConfig& c = *cfg;
    TSHIP_REQUIRE(c.n_layers > 0 && c.hidden > 0 && c.n_heads > 0 && c.n_kv_heads > 0 && c.vocab > 0, "TSHip_GptCreate: sizes must be positive");
    TSHIP_REQUIRE(c.hidden % c.n_heads == 0, "TSHip_GptCreate: hidden must be divisible by n_heads");
    TSHIP_REQUIRE(c.n_heads % c.n_kv_heads == 0, "TSHip_GptCreate: n_heads must be divisible by n_kv_heads");
    TSHIP_REQUIRE(c.attn_type == 1 || c.n_kv_heads == c.n_heads, "TSHip_GptCreate: MultiHeadAttention needs n_kv_heads == n_heads");
    TSHIP_REQUIRE(c.hidden <= 8192, "TSHip_GptCreate: hidden up to 8192 is supported");
    TSHIP_REQUIRE(c.dtype == TSHIP_F32 || c.dtype == TSHIP_F16, "TSHip_GptCreate: dtype must be f32 or f16");
    TSHIP_REQUIRE(c.max_batch >= 1 && c.max_batch <= 128, "TSHip_GptCreate: max_batch must be in 1..128");
    TSHIP_REQUIRE(c.max_seq_len >= 2, "TSHip_GptCreate: max_seq_len too small");
    TSHIP_REQUIRE(c.act >= 0 && c.act <= 4, "TSHip_GptCreate: unknown activation");
    TSHIP_REQUIRE(c.norm_type == 0 || c.norm_type == 1, "TSHip_GptCreate: unknown norm type");
    TSHIP_REQUIRE(c.max_segments >= 0 && c.max_segments <= 65536, "TSHip_GptCreate: max_segments out of range");
    std::unique_ptr<TSHipGpt> m(new TSHipGpt());
    m->c = c;
    m->f16 = c.dtype == TSHIP_F16;
    m->D = c.hidden / c.n_heads;
    {
        // GroupQueryAttention.cs:156-159 expands the KV heads by any whole factor.  The attention kernels take up to eight
        // query heads per block: a larger factor is served as groups of its largest divisor up to eight.
        const int per_kv = c.n_heads / c.n_kv_heads;
        m->G = 1;
        for (int g = 2; g <= 8; ++g) if (per_kv % g == 0) m->G = g;
        m->SG = per_kv / m->G;
        m->Hv = c.n_kv_heads * m->SG;
    }
    TSHIP_REQUIRE(m->D == 16 || m->D == 32 || m->D == 64 || m->D == 128, "TSHip_GptCreate: head_dim must be 16, 32, 64 or 128");
    TSHIP_REQUIRE(m->SG < 32, "TSHip_GptCreate: the query heads of a KV head must split into fewer than 32 groups of up to eight (at most 248 per KV head, no large prime counts)");
    m->Nqkv = (c.n_heads + 2 * c.n_kv_heads) * m->D;
    m->BT = c.max_batch <= 32 ? 1 : (c.max_batch <= 64 ? 2 : 4);
    m->Bpad = m->BT * 32;
    m->gated = (c.act == 3 || c.act == 4);
    m->F13 = m->gated ? 2 * c.ffn_dim : c.ffn_dim;
    if (c.n_experts > 1) {
        TSHIP_REQUIRE(c.experts_per_token >= 1 && c.experts_per_token <= c.n_experts && c.n_experts <= 64, "TSHip_GptCreate: bad MoE sizes");
        TSHIP_REQUIRE(!m->gated, "TSHip_GptCreate: the reference's MoE experts are two-matrix MLPs; a gated activation has no third matrix");
    }
    const long h4 = 4L * c.hidden;
    m->ML = round_up(c.max_seq_len, 32);
    m->vt = m->f16 && (m->D == 64 || m->D == 128);
    m->ldh = round_up(c.hidden, 16);
    m->ldF = round_up(std::max<long>(c.ffn_dim, c.n_experts > 1 ? h4 : 0), 16);
    const int h = c.hidden;
    for (int i = 0; i < c.n_layers; ++i) {
        m->L.emplace_back(new LayerW());
        LayerW& L = *m->L.back();
        L.moe = c.n_experts > 1 && i > 1;      // Networks/GPTDecoder.cs:114-124
        if (L.moe) for (int e = 0; e < c.n_experts; ++e) { L.e1.emplace_back(new GemmW()); L.e2.emplace_back(new GemmW()); }
        size_t cache_bytes = (size_t)c.max_batch * c.n_kv_heads * m->ML * m->D * m->esz();
        L.kc.alloc(cache_bytes); L.vc.alloc(cache_bytes);
    }
    build_expected(m.get());
    // rotary table, computed exactly as the reference's expression (TensorApplyCPU.cs:1161-1164):
    // theta = (float)pow(base, -2 i / cols); cos/sin of the float product theta * m, evaluated in double
    if (c.use_rope) {
        const int D = m->D;
        std::vector<float> cs((size_t)c.max_seq_len * D / 2), sn(cs.size());
        for (int i = 0; i < D / 2; ++i) {
            float theta = (float)std::pow((double)c.rope_base, -2.0 * (double)i / (double)D);
            for (int p = 0; p < c.max_seq_len; ++p) {
                float tm = theta * (float)p;
                cs[(size_t)p * (D / 2) + i] = (float)std::cos((double)tm);
                sn[(size_t)p * (D / 2) + i] = (float)std::sin((double)tm);
            }
        }
        upload_f32(m->rope_cos, cs.data(), cs.size());
        upload_f32(m->rope_sin, sn.data(), sn.size());
    }
    // decode buffers
    const long hp = round_up(h, 32), qp = round_up(m->Nqkv, 32), Vp = round_up(c.vocab, 32);
    m->x.alloc((size_t)m->Bpad * h * sizeof(float));
    m->xn.alloc((size_t)m->Bpad * m->ldh * m->esz());
    m->o.alloc((size_t)m->Bpad * m->ldh * m->esz());
    m->a.alloc((size_t)m->Bpad * m->ldF * m->esz());
    m->part_qkv.alloc((size_t)16 * m->Bpad * qp * sizeof(float));
    m->part_h.alloc((size_t)16 * m->Bpad * hp * sizeof(float));
    if (!m->f16) m->part_f.alloc((size_t)16 * m->Bpad * m->F13 * sizeof(float));
    m->logits.alloc((size_t)m->Bpad * Vp * sizeof(float));
    m->ids.alloc((size_t)m->Bpad * sizeof(int));
    m->d_pos.alloc(2 * sizeof(int));      // [0] cached positions, [1] step counter of the running generate call
    if (m->vt) {
        const long pairs = (long)c.max_batch * m->Hv, per = (long)m->G * m->D + 2 * m->G;
        // at most as many blocks as CUs (or one per pair) ever share the area
        const long blocks = std::max<long>(pairs, std::min<long>(pairs * TSHipGpt::MAX_ATTN_SPLITS, 2L * n_compute_units()));
        m->attn_xchg.alloc((size_t)(blocks * per) * sizeof(float));
        m->attn_count.alloc((size_t)pairs * sizeof(int));
        TSHIP_CHECK_HIP(hipMemset(m->attn_count.p, 0, m->attn_count.bytes));
    }
    m->blocked.alloc(round_up(c.vocab, 64));
    TSHIP_CHECK_HIP(hipMemset(m->blocked.p, 0, m->blocked.bytes));
    m->hidden.alloc((size_t)m->Bpad * h * sizeof(float));
    if (c.n_experts > 1) moe_alloc(m.get());
    // (LayerNorm: batches of up to 32 rows; the tails of larger batches do not store the tiles' plain sums)
    m->fused_norm = m->f16 && c.n_experts <= 1 && (c.norm_type == 0 || m->BT == 1);
    m->ln = m->fused_norm && c.norm_type == 1;
    if (m->fused_norm) {
        m->ssq.alloc((size_t)(m->ln ? 2 : 1) * (hp / 32) * m->Bpad * sizeof(float));
        m->tile_count.alloc((size_t)(std::max<long>(hp, round_up(m->F13, 32)) / 32) * sizeof(int));     // zero-filled; every use returns it to zero
    }
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    *out = m.release();
    TSHIP_END
}

TSHIP_API int TSHip_GptDestroy(TSHipGpt* m) {
    TSHIP_BEGIN
    if (m) {
        (void)hipStreamSynchronize(stream());
        if (m->step_graph) (void)hipGraphExecDestroy(m->step_graph);
        delete m;
    }
    TSHIP_END
}

TSHIP_API int TSHip_GptSetWeight(TSHipGpt* m, const char* name, const float* host_data, int ndim, const int64_t* sizes) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m && name && host_data && sizes, "TSHip_GptSetWeight: null argument");
    TSHIP_REQUIRE(ndim >= 1 && ndim <= 3, "TSHip_GptSetWeight: ndim must be 1..3");
    set_weight(m, name, host_data, ndim, sizes);
    TSHIP_END
}

TSHIP_API int TSHip_GptFinalize(TSHipGpt* m) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m, "TSHip_GptFinalize: null model");
    for (auto& n : m->expected)
        if (!m->seen.count(n)) throw Error("TSHip_GptFinalize: weight '" + n + "' was never set");
    // RMSNorm has no beta (Layers/RMSNormalization.cs:33-37): keep null pointers there
    if (m->fused_norm) {
        // deferred-norm path: the output projection runs unsplit with the residual tail in its epilogue; the FFN down
        // projection keeps its K split only when K is long enough to need more than two passes per wavefront
        for (auto& L : m->L) {
            // residual-tail projections (N = hidden): split K so that the launch has about one block per compute unit
            // (more blocks than that run in a second wave, which measured 2 us slower); BT > 1 keeps them unsplit
            auto tail_ks = [&](const GemmW& w) {
                if (m->BT != 1) return 1;
                int ks = std::max(1, n_compute_units() / std::max(1, w.NT));
                ks = std::min(ks, std::max(1, w.KT / 8));           // at least one k-tile per wavefront
                return std::min(ks, 16);
            };
            L->wo.KS = tail_ks(L->wo);
            L->w2.KS = m->BT == 1 ? tail_ks(L->w2) : (L->w2.KS <= 2 ? 1 : L->w2.KS);
        }
    }
    if (m->ln) {
        // deferred LayerNorm: every consumer of a normalised row gets the norm's gamma and beta folded through its weights
        // (LayerNormalization.Norm feeds Q/K/V or QKV, feedForwardLayer1/3 and the vocabulary projection)
        auto fold = [&](DevBuf& dst, const GemmW& w, const DevBuf& gamma, const DevBuf& beta, const float* b1, const float* b2, int mode, int n_logical) {
            const long n_packed = (long)w.NT * 32;
            dst.alloc((size_t)2 * n_packed * sizeof(float));
            ln_fold_kernel<<<(unsigned)ceil_div(n_packed, 64), 64, 0, stream()>>>(w.buf.as<half_t>(), w.KT, w.NT, w.K, gamma.as<float>(), beta.as<float>(), b1, b2, mode, n_logical,
                                                                                   dst.as<float>() + n_packed, dst.as<float>());
            TSHIP_CHECK_HIP(hipGetLastError());
        };
        const int F = m->c.ffn_dim;
        for (int l = 0; l < m->c.n_layers; ++l) {
            LayerW& L = *m->L[l];
            TSHIP_REQUIRE((long)L.qkv.NT * 32 == round_up(m->Nqkv, 32), "internal: QKV tile count");
            fold(L.ln_qkv, L.qkv, L.n1_g, L.n1_b, L.bqkv.as<float>(), nullptr, 0, m->Nqkv);
            fold(L.ln_13, L.w13, L.n2_g, L.n2_b, L.b1.as<float>(), L.b3.as<float>(), m->gated ? 1 : 0, F);
        }
        fold(m->ln_head, m->head, m->fn_g, m->fn_b, m->head_b.as<float>(), nullptr, 0, m->c.vocab);
        TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    }
    for (auto& L : m->L) {
        if (!L->moe) continue;
        const int E = m->c.n_experts, k = m->c.experts_per_token;
        L->route.alloc((size_t)m->Bpad * (E + 2 * k) * sizeof(float));
        if (!m->f16) continue;
        std::vector<const void*> t1(E), t2(E);
        for (int e = 0; e < E; ++e) { t1[e] = L->e1[e]->buf.p; t2[e] = L->e2[e]->buf.p; }
        L->wtab1.alloc(E * sizeof(void*)); L->wtab2.alloc(E * sizeof(void*));
        TSHIP_CHECK_HIP(hipMemcpyAsync(L->wtab1.p, t1.data(), E * sizeof(void*), hipMemcpyHostToDevice, stream()));
        TSHIP_CHECK_HIP(hipMemcpyAsync(L->wtab2.p, t2.data(), E * sizeof(void*), hipMemcpyHostToDevice, stream()));
        TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));       // (the host tables are locals)
    }
    m->finalized = true;
    TSHIP_END
}

TSHIP_API int TSHip_GptReset(TSHipGpt* m) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m, "TSHip_GptReset: null model");
    m->pos = 0; m->cur_batch = 0;
    TSHIP_CHECK_HIP(hipMemsetAsync(m->d_pos.p, 0, sizeof(int), stream()));
    if (m->tile_count.p) TSHIP_CHECK_HIP(hipMemsetAsync(m->tile_count.p, 0, m->tile_count.bytes, stream()));
    if (m->last_pos.p) TSHIP_CHECK_HIP(hipMemsetAsync(m->last_pos.p, 0xff, m->last_pos.bytes, stream()));      // -1: no token seen
    if (m->attn_count.p) TSHIP_CHECK_HIP(hipMemsetAsync(m->attn_count.p, 0, m->attn_count.bytes, stream()));
    if (m->moe_ws.p) TSHIP_CHECK_HIP(hipMemsetAsync((char*)m->moe_ws.p + moe_layout(m, m->Bpad).counts, 0, (size_t)m->c.n_experts * sizeof(int), stream()));
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    TSHIP_END
}

TSHIP_API int TSHip_GptSetBlockedTokens(TSHipGpt* m, const int32_t* ids, int n) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m && (ids || n == 0) && n >= 0, "TSHip_GptSetBlockedTokens: bad argument");
    std::vector<unsigned char> mask(m->blocked.bytes, 0);
    for (int i = 0; i < n; ++i) {
        TSHIP_REQUIRE(ids[i] >= 0 && ids[i] < m->c.vocab, "TSHip_GptSetBlockedTokens: token id out of range");
        mask[ids[i]] = 1;
    }
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    TSHIP_CHECK_HIP(hipMemcpy(m->blocked.p, mask.data(), mask.size(), hipMemcpyHostToDevice));
    // the choice kernels only look at the list when there is one; a captured step carries that decision
    if ((n > 0) != m->any_blocked && m->step_graph) { (void)hipGraphExecDestroy(m->step_graph); m->step_graph = nullptr; }
    m->any_blocked = n > 0;
    TSHIP_END
}

TSHIP_API int TSHip_GptSetRepeatPenalty(TSHipGpt* m, float repeat_penalty) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m, "TSHip_GptSetRepeatPenalty: null model");
    TSHIP_REQUIRE(std::isfinite(repeat_penalty), "TSHip_GptSetRepeatPenalty: the penalty must be finite");
    if (repeat_penalty != 0.0f && !m->last_pos.p) {
        TSHIP_REQUIRE(m->pos == 0, "TSHip_GptSetRepeatPenalty: sequences are under way; set the penalty before the prompt is fed or after TSHip_GptReset");
        m->last_ld = round_up(m->c.vocab, 64);
        m->last_pos.alloc((size_t)m->c.max_batch * m->last_ld * sizeof(int));
        TSHIP_CHECK_HIP(hipMemsetAsync(m->last_pos.p, 0xff, m->last_pos.bytes, stream()));
        TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    }
    m->repeat_penalty = repeat_penalty;
    TSHIP_END
}

TSHIP_API int TSHip_GptPrefill(TSHipGpt* m, const int32_t* host_ids, int batch, int prompt_len) {
    TSHIP_BEGIN
    refresh_test_hooks();
    TSHIP_REQUIRE(m && host_ids, "TSHip_GptPrefill: null argument");
    TSHIP_REQUIRE(m->finalized, "TSHip_GptPrefill: call TSHip_GptFinalize first");
    TSHIP_REQUIRE(batch >= 1 && batch <= m->c.max_batch, "TSHip_GptPrefill: batch out of range");
    for (long i = 0; i < (long)batch * prompt_len; ++i)
        TSHIP_REQUIRE(host_ids[i] >= 0 && host_ids[i] < m->c.vocab, "TSHip_GptPrefill: token id out of range");
    prefill(m, host_ids, batch, prompt_len);
    TSHIP_END
}

TSHIP_API int TSHip_GptPrefillPadded(TSHipGpt* m, const int32_t* host_ids, const int32_t* host_lens, int batch, int padded_len) {
    TSHIP_BEGIN
    refresh_test_hooks();
    TSHIP_REQUIRE(m && host_ids && host_lens, "TSHip_GptPrefillPadded: null argument");
    TSHIP_REQUIRE(m->finalized, "TSHip_GptPrefillPadded: call TSHip_GptFinalize first");
    TSHIP_REQUIRE(batch >= 1 && batch <= m->c.max_batch, "TSHip_GptPrefillPadded: batch out of range");
    for (int b = 0; b < batch; ++b) TSHIP_REQUIRE(host_lens[b] >= 0 && host_lens[b] <= padded_len, "TSHip_GptPrefillPadded: a sequence length lies outside 0..padded_len");
    for (long i = 0; i < (long)batch * padded_len; ++i)
        TSHIP_REQUIRE(host_ids[i] >= 0 && host_ids[i] < m->c.vocab, "TSHip_GptPrefillPadded: token id out of range");
    prefill(m, host_ids, batch, padded_len, host_lens);
    TSHIP_END
}

TSHIP_API int TSHip_GptDecode(TSHipGpt* m, const int32_t* host_ids, int batch) {
    TSHIP_BEGIN
    refresh_test_hooks();
    TSHIP_REQUIRE(m && host_ids, "TSHip_GptDecode: null argument");
    TSHIP_REQUIRE(m->finalized, "TSHip_GptDecode: call TSHip_GptFinalize first");
    TSHIP_REQUIRE(batch >= 1 && batch <= m->c.max_batch, "TSHip_GptDecode: batch out of range");
    TSHIP_REQUIRE(m->cur_batch == 0 || m->cur_batch == batch, "TSHip_GptDecode: batch differs from the cached sequences");
    TSHIP_REQUIRE(m->pos + 1 <= m->c.max_seq_len, "TSHip_GptDecode: KV cache is full (max_seq_len)");
    for (int i = 0; i < batch; ++i) TSHIP_REQUIRE(host_ids[i] >= 0 && host_ids[i] < m->c.vocab, "TSHip_GptDecode: token id out of range");
    TSHIP_CHECK_HIP(hipMemcpyAsync(m->ids.p, host_ids, batch * sizeof(int), hipMemcpyHostToDevice, stream()));
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    m->embed_done = false;          // (set only between a sampling kernel and the decode step that follows it at once)
    record_history(m, m->ids.as<int>(), batch, 1, m->pos);
    decode_step(m, m->ids.as<int>(), batch);
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    m->cur_batch = batch;
    TSHIP_END
}

TSHIP_API int TSHip_GptSample(TSHipGpt* m, int mode, float top_p, float temperature, const float* host_uniforms, int32_t* host_ids_out) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m && host_ids_out, "TSHip_GptSample: null argument");
    TSHIP_REQUIRE(m->cur_batch > 0, "TSHip_GptSample: no logits yet; prefill or decode first");
    const int B = m->cur_batch;
    sample_tokens(m, mode, top_p, temperature, host_uniforms, nullptr, B, nullptr, nullptr, false);
    TSHIP_CHECK_HIP(hipMemcpyAsync(host_ids_out, m->ids.p, B * sizeof(int), hipMemcpyDeviceToHost, stream()));
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    TSHIP_END
}

// the token loop; eos_id >= 0: the host looks at every step's tokens and stops after the first step whose tokens are
// all eos_id (Decoder.AreAllSentsCompleted, Applications/Decoder.cs:207-221, as GPT.cs:299-302 uses it)
static int generate_impl(TSHipGpt* m, int n_steps, int mode, float top_p, float temperature, const float* host_uniforms, int32_t* host_ids_out,
                         float* elapsed_ms, int eos_id, int* steps_done) {
    TSHIP_BEGIN
    refresh_test_hooks();
    TSHIP_REQUIRE(m && host_ids_out, "TSHip_GptGenerate: null argument");
    TSHIP_REQUIRE(m->cur_batch > 0, "TSHip_GptGenerate: no logits yet; prefill first");
    TSHIP_REQUIRE(n_steps >= 1, "TSHip_GptGenerate: n_steps must be positive");
    TSHIP_REQUIRE(m->pos + n_steps <= m->c.max_seq_len, "TSHip_GptGenerate: KV cache too small for n_steps (max_seq_len)");
    m->embed_done = false;
    TSHIP_REQUIRE(mode == TSHIP_GREEDY || (mode == TSHIP_TOPP && host_uniforms), "TSHip_GptGenerate: top-p needs the uniform stream");
    const int B = m->cur_batch;
    // token and uniform buffers live in the model so that the captured step graph stays valid across calls
    DevBuf& gen = m->gen_buf; DevBuf& uni = m->uni_buf;
    if (gen.bytes < (size_t)n_steps * B * sizeof(int)) gen.alloc((size_t)std::max(n_steps, 256) * m->Bpad * sizeof(int));
    if (mode == TSHIP_TOPP) {
        if (uni.bytes < (size_t)n_steps * B * sizeof(float)) uni.alloc((size_t)std::max(n_steps, 256) * m->Bpad * sizeof(float));
        TSHIP_CHECK_HIP(hipMemcpyAsync(uni.p, host_uniforms, (size_t)n_steps * B * sizeof(float), hipMemcpyHostToDevice, stream()));
        TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    }
    // the step counter that indexes gen/uniforms on the device starts at zero for every call
    TSHIP_CHECK_HIP(hipMemsetAsync(m->d_pos.as<int>() + 1, 0, sizeof(int), stream()));
    const int* d_step = m->d_pos.as<int>() + 1;
    const float* uni_base = mode == TSHIP_TOPP ? uni.as<float>() : nullptr;
    const bool use_graph = !g_hooks.no_graph;
    if (mode == TSHIP_TOPP) {      // scratch must exist before capture (no allocation inside a graph)
        const size_t need = topp_scratch_bytes(m->Bpad, m->c.vocab);
        if (m->topp_scratch.bytes < need) m->topp_scratch.alloc(need);
    }
    if (use_graph) {
        // (sample -> decode) of one step is captured once; every replay reads the position, the step counter and the
        // token ids from device memory, so identical launches walk through the sequence
        if (m->step_graph && (m->graph_batch != B || m->graph_mode != mode || m->graph_top_p != top_p || m->graph_temp != temperature ||
                              m->graph_uniforms != uni_base || m->graph_gen != gen.as<int>() || m->graph_penalty != m->repeat_penalty)) {
            (void)hipGraphExecDestroy(m->step_graph); m->step_graph = nullptr;
        }
        if (!m->step_graph) {
            hipGraph_t graph = nullptr;
            // the arrival counters of the one-launch reductions are zero between launches; a step that ended in an error
            // may have left them otherwise, and every replay of the graph starts from what is there
            if (m->tile_count.p) TSHIP_CHECK_HIP(hipMemsetAsync(m->tile_count.p, 0, m->tile_count.bytes, stream()));
            if (m->attn_count.p) TSHIP_CHECK_HIP(hipMemsetAsync(m->attn_count.p, 0, m->attn_count.bytes, stream()));
            TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
            TSHIP_CHECK_HIP(hipStreamBeginCapture(stream(), hipStreamCaptureModeThreadLocal));
            const int saved_pos = m->pos;
            try {
                sample_tokens(m, mode, top_p, temperature, nullptr, uni_base, B, gen.as<int>(), d_step, true, true);
                decode_step(m, m->ids.as<int>(), B);
            } catch (...) { hipGraph_t g2 = nullptr; (void)hipStreamEndCapture(stream(), &g2); if (g2) (void)hipGraphDestroy(g2); m->pos = saved_pos; m->embed_done = false; throw; }
            m->pos = saved_pos;                    // capturing launched nothing
            TSHIP_CHECK_HIP(hipStreamEndCapture(stream(), &graph));
            hipError_t ge = hipGraphInstantiate(&m->step_graph, graph, nullptr, nullptr, 0);
            (void)hipGraphDestroy(graph);
            TSHIP_CHECK_HIP(ge);
            m->graph_batch = B; m->graph_mode = mode; m->graph_top_p = top_p; m->graph_temp = temperature;
            m->graph_uniforms = uni_base; m->graph_gen = gen.as<int>(); m->graph_penalty = m->repeat_penalty;
        }
    }
    struct EventPair {      // destroyed on every path out of the function
        hipEvent_t a = nullptr, b = nullptr;
        ~EventPair() { if (a) (void)hipEventDestroy(a); if (b) (void)hipEventDestroy(b); }
    } ev;
    TSHIP_CHECK_HIP(hipEventCreate(&ev.a));
    TSHIP_CHECK_HIP(hipEventCreate(&ev.b));
    const hipEvent_t e0 = ev.a, e1 = ev.b;
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    TSHIP_CHECK_HIP(hipEventRecord(e0, stream()));
    int done = 0;
    for (int s = 0; s < n_steps; ++s) {
        if (use_graph) { TSHIP_CHECK_HIP(hipGraphLaunch(m->step_graph, stream())); m->pos += 1; }
        else {
            sample_tokens(m, mode, top_p, temperature, nullptr, uni_base, B, gen.as<int>(), d_step, true, true);
            decode_step(m, m->ids.as<int>(), B);
        }
        done = s + 1;
        if (eos_id >= 0) {
            // (one small copy and a synchronisation per step: the price of looking at the tokens on the host)
            TSHIP_CHECK_HIP(hipMemcpyAsync(host_ids_out + (size_t)s * B, gen.as<int>() + (size_t)s * B, (size_t)B * sizeof(int), hipMemcpyDeviceToHost, stream()));
            TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
            bool all_eos = true;
            for (int b = 0; b < B; ++b) all_eos = all_eos && host_ids_out[(size_t)s * B + b] == eos_id;
            if (all_eos) break;
        }
    }
    TSHIP_CHECK_HIP(hipEventRecord(e1, stream()));
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    float ms = 0.0f;
    TSHIP_CHECK_HIP(hipEventElapsedTime(&ms, e0, e1));
    if (elapsed_ms) *elapsed_ms = ms;
    if (steps_done) *steps_done = done;
    if (eos_id < 0) TSHIP_CHECK_HIP(hipMemcpy(host_ids_out, gen.p, (size_t)n_steps * B * sizeof(int), hipMemcpyDeviceToHost));
    TSHIP_END
}

TSHIP_API int TSHip_GptGenerate(TSHipGpt* m, int n_steps, int mode, float top_p, float temperature,
                                const float* host_uniforms, int32_t* host_ids_out, float* elapsed_ms) {
    return generate_impl(m, n_steps, mode, top_p, temperature, host_uniforms, host_ids_out, elapsed_ms, -1, nullptr);
}

TSHIP_API int TSHip_GptGenerateUntil(TSHipGpt* m, int max_steps, int eos_id, int mode, float top_p, float temperature,
                                     const float* host_uniforms, int32_t* host_ids_out, int* steps_done, float* elapsed_ms) {
    if (m && (eos_id < 0 || eos_id >= m->c.vocab)) { set_last_error("TSHip_GptGenerateUntil: eos_id out of range"); return 0; }
    if (!steps_done) { set_last_error("TSHip_GptGenerateUntil: null argument"); return 0; }
    return generate_impl(m, max_steps, mode, top_p, temperature, host_uniforms, host_ids_out, elapsed_ms, eos_id, steps_done);
}

TSHIP_API int TSHip_GptBeamPick(TSHipGpt* m, int n_picks, int mode, float top_p, float temperature, const float* host_uniforms,
                                int32_t* host_ids_out, float* host_logp_out) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m && host_ids_out && host_logp_out, "TSHip_GptBeamPick: null argument");
    TSHIP_REQUIRE(m->cur_batch > 0, "TSHip_GptBeamPick: no logits yet; prefill or decode first");
    TSHIP_REQUIRE(n_picks >= 1 && n_picks <= m->c.vocab, "TSHip_GptBeamPick: n_picks must lie in 1..vocab");
    TSHIP_REQUIRE(mode == TSHIP_GREEDY || (mode == TSHIP_TOPP && host_uniforms), "TSHip_GptBeamPick: top-p needs one uniform draw per row and pick");
    TSHIP_REQUIRE(mode == TSHIP_GREEDY || m->c.vocab <= 262144, "top-p sampling supports vocabularies up to 262144");
    TSHIP_REQUIRE(temperature > 0.0f, "temperature must be positive");
    const int B = m->cur_batch, V = m->c.vocab;
    const long Vp = round_up(V, 32);
    m->beam_probs.reserve((size_t)m->Bpad * Vp * sizeof(float));
    m->beam_ids.reserve((size_t)m->Bpad * sizeof(int));
    m->beam_out.reserve((size_t)n_picks * B * (sizeof(int) + sizeof(float)));
    int* d_ids_out = m->beam_out.as<int>(); float* d_logp = (float*)(d_ids_out + (size_t)n_picks * B);
    float* probs = m->beam_probs.as<float>();
    // Decoder.cs:720-723: the logits are divided by the temperature only when sampling
    launch(m, "beam_probs", beam_probs_kernel, dim3(B), dim3(1024), (const float*)m->logits.as<float>(), Vp, V, temperature,
           (int)(mode == TSHIP_TOPP && temperature != 1.0f), probs, Vp);
    const unsigned char* blocked = m->any_blocked ? (const unsigned char*)m->blocked.p : nullptr;
    if (mode == TSHIP_TOPP) {
        m->beam_uni.reserve((size_t)n_picks * B * sizeof(float));
        TSHIP_CHECK_HIP(hipMemcpyAsync(m->beam_uni.p, host_uniforms, (size_t)n_picks * B * sizeof(float), hipMemcpyHostToDevice, stream()));
        const size_t need = topp_scratch_bytes(m->Bpad, V);
        if (m->topp_scratch.bytes < need) m->topp_scratch.alloc(need);
    }
    for (int i = 0; i < n_picks; ++i) {
        if (mode == TSHIP_GREEDY) {
            // Argmax over the probabilities, first maximum (TensorApplyCPU.cs:339-360); nothing is recorded: the caller decides
            // which picks survive
            launch(m, "beam_argmax", greedy_kernel, dim3(B), dim3(1024), (const float*)probs, Vp, V, m->beam_ids.as<int>(), (int*)nullptr, (const int*)nullptr,
                   (int*)nullptr, 0L, (const int*)nullptr, blocked);
        } else {
            TopPArgs a; std::memset(&a, 0, sizeof(a));
            a.in = probs; a.ld = Vp; a.V = V; a.in_is_logits = 0; a.temperature = 1.0f;
            a.uniforms = m->beam_uni.as<float>() + (size_t)i * B; a.top_p = top_p;
            topp_carve(a, m->topp_scratch.p, m->Bpad, V);
            a.next_ids = m->beam_ids.as<int>();
            a.blocked = blocked;
            a.repeat_penalty = m->repeat_penalty; a.last_pos = m->last_pos.as<int>(); a.last_ld = m->last_ld; a.d_len = m->d_pos.as<int>(); a.record = 0;
            topp_run(a, B, [&](const char* name, void (*kernel)(TopPArgs), dim3 grid, dim3 block, const TopPArgs& args) { launch(m, name, kernel, grid, block, args); });
        }
        launch(m, "beam_take", beam_take_kernel, dim3((unsigned)ceil_div(B, 64)), dim3(64), probs, Vp, (const int*)m->beam_ids.as<int>(), B,
               d_ids_out + (size_t)i * B, d_logp + (size_t)i * B);
    }
    TSHIP_CHECK_HIP(hipMemcpyAsync(host_ids_out, d_ids_out, (size_t)n_picks * B * sizeof(int), hipMemcpyDeviceToHost, stream()));
    TSHIP_CHECK_HIP(hipMemcpyAsync(host_logp_out, d_logp, (size_t)n_picks * B * sizeof(float), hipMemcpyDeviceToHost, stream()));
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    TSHIP_END
}

TSHIP_API int TSHip_GptReorderRows(TSHipGpt* m, const int32_t* host_src_rows, int new_batch) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m && host_src_rows, "TSHip_GptReorderRows: null argument");
    TSHIP_REQUIRE(m->cur_batch > 0, "TSHip_GptReorderRows: no cached sequences");
    TSHIP_REQUIRE(new_batch >= 1 && new_batch <= m->c.max_batch, "TSHip_GptReorderRows: new batch out of range (max_batch)");
    bool identity = new_batch == m->cur_batch;
    for (int i = 0; i < new_batch; ++i) {
        TSHIP_REQUIRE(host_src_rows[i] >= 0 && host_src_rows[i] < m->cur_batch, "TSHip_GptReorderRows: source row out of range");
        identity = identity && host_src_rows[i] == i;
    }
    if (!identity) {
        m->reorder_src.reserve((size_t)m->c.max_batch * sizeof(int));
        TSHIP_CHECK_HIP(hipMemcpyAsync(m->reorder_src.p, host_src_rows, (size_t)new_batch * sizeof(int), hipMemcpyHostToDevice, stream()));
        TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));       // (the caller's array may go away)
        // cache rows: [batch][kv head][ML * D] elements; the first round_up(pos, 32) positions of every head are live
        // (fragment-major caches keep positions in chunks of 32)
        const long head_bytes = (long)m->ML * m->D * (long)m->esz(), row_bytes = head_bytes * m->c.n_kv_heads;
        const long used = std::min<long>(head_bytes, round_up(std::max(m->pos, 1), 32) * (long)m->D * (long)m->esz());
        m->reorder_tmp.reserve((size_t)std::max<long>(row_bytes, m->last_pos.p ? m->last_ld * (long)sizeof(int) : 0) * m->c.max_batch);
        const int* src = m->reorder_src.as<int>();
        auto gather = [&](void* table, long stride, long chunk, long live, long pieces) {
            launch(m, "rows_gather", rows_gather_kernel, dim3((unsigned)pieces, (unsigned)new_batch), dim3(256), (const char*)table, stride, chunk, live, src, m->reorder_tmp.as<char>(), 1);
            launch(m, "rows_gather", rows_gather_kernel, dim3((unsigned)pieces, (unsigned)new_batch), dim3(256), (const char*)table, stride, chunk, live, src, m->reorder_tmp.as<char>(), 0);
        };
        for (auto& L : m->L) { gather(L->kc.p, row_bytes, head_bytes, used, m->c.n_kv_heads); gather(L->vc.p, row_bytes, head_bytes, used, m->c.n_kv_heads); }
        if (m->last_pos.p) gather(m->last_pos.p, m->last_ld * (long)sizeof(int), m->last_ld * (long)sizeof(int), m->last_ld * (long)sizeof(int), 1);
        TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    }
    m->cur_batch = new_batch;
    TSHIP_END
}

TSHIP_API int TSHip_BeamTopN(const float* scores, int n, int top_n, int32_t* kept, int* n_kept) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(scores && kept && n_kept && n >= 0 && top_n >= 1, "TSHip_BeamTopN: bad argument");
    TopNQueue q(top_n);
    for (int i = 0; i < n; ++i) q.enqueue(TopNQueue::Item{scores[i], i});
    const auto items = q.enumerate();
    for (size_t i = 0; i < items.size(); ++i) kept[i] = items[i].index;
    *n_kept = (int)items.size();
    TSHIP_END
}

TSHIP_API int TSHip_GptGetLogits(TSHipGpt* m, float* host_out) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m && host_out, "TSHip_GptGetLogits: null argument");
    TSHIP_REQUIRE(m->cur_batch > 0, "TSHip_GptGetLogits: no logits yet");
    const long Vp = round_up(m->c.vocab, 32);
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    TSHIP_CHECK_HIP(hipMemcpy2D(host_out, (size_t)m->c.vocab * sizeof(float), m->logits.p, (size_t)Vp * sizeof(float),
                                (size_t)m->c.vocab * sizeof(float), m->cur_batch, hipMemcpyDeviceToHost));
    TSHIP_END
}

TSHIP_API int TSHip_GptGetHidden(TSHipGpt* m, float* host_out) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m && host_out, "TSHip_GptGetHidden: null argument");
    TSHIP_REQUIRE(m->cur_batch > 0, "TSHip_GptGetHidden: nothing computed yet");
    const int B = m->cur_batch, h = m->c.hidden;
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    if (m->fused_norm) {
        // the normalised hidden state is never materialised on this path: rebuild it from the residual stream
        std::vector<float> xs((size_t)B * h), gm(h);
        TSHIP_CHECK_HIP(hipMemcpy(xs.data(), m->x.p, xs.size() * sizeof(float), hipMemcpyDeviceToHost));
        TSHIP_CHECK_HIP(hipMemcpy(gm.data(), m->fn_g.p, gm.size() * sizeof(float), hipMemcpyDeviceToHost));
        std::vector<float> bt(h, 0.0f);
        if (m->ln) TSHIP_CHECK_HIP(hipMemcpy(bt.data(), m->fn_b.p, bt.size() * sizeof(float), hipMemcpyDeviceToHost));
        for (int b = 0; b < B; ++b) {
            double sq = 0.0, sm = 0.0;
            for (int i = 0; i < h; ++i) { sq += (double)xs[(size_t)b * h + i] * xs[(size_t)b * h + i]; sm += xs[(size_t)b * h + i]; }
            if (m->ln) {
                const double mean = sm / h;
                double d2 = 0.0;
                for (int i = 0; i < h; ++i) { const double d = xs[(size_t)b * h + i] - mean; d2 += d * d; }
                const float sigma = (float)std::sqrt(m->c.norm_eps + d2 / h);
                for (int i = 0; i < h; ++i) host_out[(size_t)b * h + i] = gm[i] * ((xs[(size_t)b * h + i] - (float)mean) / sigma) + bt[i];
                continue;
            }
            float rms = (float)std::sqrt(sq / h + m->c.norm_eps);
            for (int i = 0; i < h; ++i) host_out[(size_t)b * h + i] = gm[i] * (xs[(size_t)b * h + i] / rms);
        }
    } else if (m->f16) {
        std::vector<half_t> tmp((size_t)m->Bpad * m->ldh);
        TSHIP_CHECK_HIP(hipMemcpy(tmp.data(), m->xn.p, tmp.size() * sizeof(half_t), hipMemcpyDeviceToHost));
        const int KT = (int)(m->ldh / 16);
        for (int b = 0; b < B; ++b) for (int i = 0; i < h; ++i) {
            size_t idx = ((((size_t)(b >> 5) * KT + (i >> 4)) * 64) + (b & 31) + 32 * ((i >> 3) & 1)) * 8 + (i & 7);   // fragment packed
            host_out[(size_t)b * h + i] = (float)tmp[idx];
        }
    } else {
        TSHIP_CHECK_HIP(hipMemcpy2D(host_out, (size_t)h * sizeof(float), m->xn.p, (size_t)m->ldh * sizeof(float), (size_t)h * sizeof(float), B, hipMemcpyDeviceToHost));
    }
    TSHIP_END
}

TSHIP_API int TSHip_GptGetSeqLen(TSHipGpt* m, int* len) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m && len, "TSHip_GptGetSeqLen: null argument");
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    int dev = 0;
    TSHIP_CHECK_HIP(hipMemcpy(&dev, m->d_pos.p, sizeof(int), hipMemcpyDeviceToHost));
    TSHIP_REQUIRE(dev == m->pos, "internal: device and host sequence positions disagree");
    *len = m->pos;
    TSHIP_END
}

TSHIP_API int TSHip_GptGetKV(TSHipGpt* m, int layer, int which, float* host_out) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m && host_out, "TSHip_GptGetKV: null argument");
    TSHIP_REQUIRE(layer >= 0 && layer < m->c.n_layers && (which == 0 || which == 1), "TSHip_GptGetKV: bad layer or selector");
    const int B = m->cur_batch, G = m->c.n_kv_heads, D = m->D, T = m->pos; const long ML = m->ML;
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    const char* base = (const char*)(which ? m->L[layer]->vc.p : m->L[layer]->kc.p);
    const bool frag = m->vt;                               // fragment-major cache of the MFMA attention kernels
    std::vector<char> tmp((size_t)ML * D * m->esz());
    for (int b = 0; b < B; ++b) for (int g = 0; g < G; ++g) {
        TSHIP_CHECK_HIP(hipMemcpy(tmp.data(), base + ((size_t)b * G + g) * ML * D * m->esz(), tmp.size(), hipMemcpyDeviceToHost));
        float* dst = host_out + ((size_t)b * G + g) * T * D;
        for (long t = 0; t < T; ++t) for (int d = 0; d < D; ++d) {
            size_t idx = frag ? (size_t)(which ? vfrag_index((int)t, d, D) : kfrag_index((int)t, d, D)) : (size_t)t * D + d;
            dst[t * D + d] = m->f16 ? (float)((const half_t*)tmp.data())[idx] : ((const float*)tmp.data())[idx];
        }
    }
    TSHIP_END
}

TSHIP_API int TSHip_GptSetSeqLen(TSHipGpt* m, int batch, int len) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m, "TSHip_GptSetSeqLen: null model");
    TSHIP_REQUIRE(batch >= 1 && batch <= m->c.max_batch && len >= 0 && len < m->c.max_seq_len, "TSHip_GptSetSeqLen: out of range");
    m->pos = len; m->cur_batch = batch;
    TSHIP_CHECK_HIP(hipMemcpyAsync(m->d_pos.p, &m->pos, sizeof(int), hipMemcpyHostToDevice, stream()));
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    TSHIP_END
}

TSHIP_API int TSHip_GptSetKV(TSHipGpt* m, int layer, int which, const float* host_in, int batch, int len) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m && host_in, "TSHip_GptSetKV: null argument");
    TSHIP_REQUIRE(layer >= 0 && layer < m->c.n_layers && (which == 0 || which == 1), "TSHip_GptSetKV: bad layer or selector");
    TSHIP_REQUIRE(batch >= 1 && batch <= m->c.max_batch && len >= 0 && len <= m->c.max_seq_len, "TSHip_GptSetKV: out of range");
    const int G = m->c.n_kv_heads, D = m->D; const long ML = m->ML;
    char* base = (char*)(which ? m->L[layer]->vc.p : m->L[layer]->kc.p);
    const bool frag = m->vt;
    std::vector<char> tmp((size_t)ML * D * m->esz(), 0);
    for (int b = 0; b < batch; ++b) for (int g = 0; g < G; ++g) {
        const float* src = host_in + ((size_t)b * G + g) * len * D;
        for (long t = 0; t < len; ++t) for (int d = 0; d < D; ++d) {
            size_t idx = frag ? (size_t)(which ? vfrag_index((int)t, d, D) : kfrag_index((int)t, d, D)) : (size_t)t * D + d;
            if (m->f16) ((half_t*)tmp.data())[idx] = (half_t)src[t * D + d]; else ((float*)tmp.data())[idx] = src[t * D + d];
        }
        TSHIP_CHECK_HIP(hipMemcpy(base + ((size_t)b * G + g) * ML * D * m->esz(), tmp.data(), tmp.size(), hipMemcpyHostToDevice));
    }
    TSHIP_END
}

// ------------------------------------------------------------------------------------------------
// Saved sequence sets.  The reference keeps the KV tensors of finished requests in a MemoryCache keyed by the generated
// text (10 minutes sliding expiry) and puts them back when a request continues that text
// (Seq2SeqSharp/Applications/GPT.cs:153-173, 236-247, 312-328).  Here the cache rows stay on the device: a snapshot holds
// the used prefix of the model's cache regions; the text-keyed dictionary lives with the caller.
// ------------------------------------------------------------------------------------------------
static size_t used_region_bytes(const TSHipGpt* m, int len) {
    // fragment-major layout: whole 32-position chunks; row-major: whole positions
    const long rows = m->vt ? round_up(len, 32) : len;
    return (size_t)rows * m->D * m->esz();
}

TSHIP_API int TSHip_GptSaveRows(TSHipGpt* m, TSHipGptSnapshot** out) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m && out, "TSHip_GptSaveRows: null argument");
    TSHIP_REQUIRE(m->finalized && m->cur_batch > 0, "TSHip_GptSaveRows: no sequences in the cache (prefill first)");
    std::unique_ptr<TSHipGptSnapshot> sn(new TSHipGptSnapshot());
    const int B = m->cur_batch, G = m->c.n_kv_heads;
    sn->batch = B; sn->len = m->pos; sn->n_layers = m->c.n_layers; sn->n_kv_heads = G; sn->D = m->D; sn->vocab = m->c.vocab;
    sn->f16 = m->f16; sn->vt = m->vt;
    sn->region_bytes = used_region_bytes(m, m->pos);
    const size_t pitch = (size_t)m->ML * m->D * m->esz();
    for (int l = 0; l < m->c.n_layers; ++l) {
        sn->k.emplace_back(new DevBuf()); sn->v.emplace_back(new DevBuf());
        if (sn->region_bytes == 0) continue;
        sn->k[l]->alloc(sn->region_bytes * B * G); sn->v[l]->alloc(sn->region_bytes * B * G);
        TSHIP_CHECK_HIP(hipMemcpy2DAsync(sn->k[l]->p, sn->region_bytes, m->L[l]->kc.p, pitch, sn->region_bytes, (size_t)B * G, hipMemcpyDeviceToDevice, stream()));
        TSHIP_CHECK_HIP(hipMemcpy2DAsync(sn->v[l]->p, sn->region_bytes, m->L[l]->vc.p, pitch, sn->region_bytes, (size_t)B * G, hipMemcpyDeviceToDevice, stream()));
        sn->total_bytes += 2 * sn->region_bytes * B * G;
    }
    const size_t lbytes = (size_t)B * round_up(m->c.vocab, 32) * sizeof(float);
    sn->logits.alloc(lbytes);
    TSHIP_CHECK_HIP(hipMemcpyAsync(sn->logits.p, m->logits.p, lbytes, hipMemcpyDeviceToDevice, stream()));
    sn->total_bytes += lbytes;
    if (m->last_pos.p) {
        sn->last_ld = m->last_ld;
        const size_t hbytes = (size_t)B * m->last_ld * sizeof(int);
        sn->last_pos.alloc(hbytes);
        TSHIP_CHECK_HIP(hipMemcpyAsync(sn->last_pos.p, m->last_pos.p, hbytes, hipMemcpyDeviceToDevice, stream()));
        sn->total_bytes += hbytes;
    }
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    *out = sn.release();
    TSHIP_END
}

TSHIP_API int TSHip_GptRestoreRows(TSHipGpt* m, const TSHipGptSnapshot* sn) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m && sn, "TSHip_GptRestoreRows: null argument");
    TSHIP_REQUIRE(m->finalized, "TSHip_GptRestoreRows: the model is not finalised");
    TSHIP_REQUIRE(sn->n_layers == m->c.n_layers && sn->n_kv_heads == m->c.n_kv_heads && sn->D == m->D && sn->vocab == m->c.vocab &&
                  sn->f16 == m->f16 && sn->vt == m->vt, "TSHip_GptRestoreRows: the snapshot was taken from a model of another shape or type");
    TSHIP_REQUIRE(sn->batch <= m->c.max_batch && sn->len < m->c.max_seq_len, "TSHip_GptRestoreRows: the snapshot does not fit this model's cache");
    TSHIP_REQUIRE(!m->last_pos.p || (sn->last_pos.p && sn->last_ld == m->last_ld),
                  "TSHip_GptRestoreRows: the model keeps a token history (repeat penalty) and the snapshot holds none");
    const int B = sn->batch, G = sn->n_kv_heads;
    const size_t pitch = (size_t)m->ML * m->D * m->esz();
    TSHIP_REQUIRE(sn->region_bytes <= pitch, "TSHip_GptRestoreRows: the snapshot's regions are longer than this model's");
    for (int l = 0; l < m->c.n_layers && sn->region_bytes; ++l) {
        TSHIP_CHECK_HIP(hipMemcpy2DAsync(m->L[l]->kc.p, pitch, sn->k[l]->p, sn->region_bytes, sn->region_bytes, (size_t)B * G, hipMemcpyDeviceToDevice, stream()));
        TSHIP_CHECK_HIP(hipMemcpy2DAsync(m->L[l]->vc.p, pitch, sn->v[l]->p, sn->region_bytes, sn->region_bytes, (size_t)B * G, hipMemcpyDeviceToDevice, stream()));
    }
    TSHIP_CHECK_HIP(hipMemcpyAsync(m->logits.p, sn->logits.p, sn->logits.bytes, hipMemcpyDeviceToDevice, stream()));
    if (m->last_pos.p) TSHIP_CHECK_HIP(hipMemcpyAsync(m->last_pos.p, sn->last_pos.p, (size_t)B * m->last_ld * sizeof(int), hipMemcpyDeviceToDevice, stream()));
    m->pos = sn->len; m->cur_batch = B; m->embed_done = false;
    TSHIP_CHECK_HIP(hipMemcpyAsync(m->d_pos.p, &m->pos, sizeof(int), hipMemcpyHostToDevice, stream()));
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    TSHIP_END
}

TSHIP_API int TSHip_GptSnapshotInfo(const TSHipGptSnapshot* sn, int* batch, int* len, int64_t* device_bytes) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(sn, "TSHip_GptSnapshotInfo: null snapshot");
    if (batch) *batch = sn->batch;
    if (len) *len = sn->len;
    if (device_bytes) *device_bytes = (int64_t)sn->total_bytes;
    TSHIP_END
}

TSHIP_API int TSHip_GptFreeSnapshot(TSHipGptSnapshot* sn) {
    TSHIP_BEGIN
    delete sn;
    TSHIP_END
}

TSHIP_API int TSHip_GptGetMoeRouting(TSHipGpt* m, int layer, float* top_idx, float* top_val, float* probs) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m, "TSHip_GptGetMoeRouting: null model");
    TSHIP_REQUIRE(layer >= 0 && layer < m->c.n_layers && m->L[layer]->moe, "TSHip_GptGetMoeRouting: not an MoE layer");
    moe_get_routing(m, layer, top_idx, top_val, probs);
    TSHIP_END
}

TSHIP_API int TSHip_GptProfileDecode(TSHipGpt* m, const int32_t* host_ids, int batch, char* names, float* ms, int n_max, int* n) {
    TSHIP_BEGIN
    refresh_test_hooks();
    TSHIP_REQUIRE(m && host_ids && names && ms && n, "TSHip_GptProfileDecode: null argument");
    TSHIP_REQUIRE(m->finalized && batch >= 1 && batch <= m->c.max_batch, "TSHip_GptProfileDecode: bad state or batch");
    TSHIP_REQUIRE(m->pos + 1 <= m->c.max_seq_len, "TSHip_GptProfileDecode: KV cache is full");
    TSHIP_CHECK_HIP(hipMemcpyAsync(m->ids.p, host_ids, batch * sizeof(int), hipMemcpyHostToDevice, stream()));
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    Profiler prof;
    m->prof = &prof;
    m->embed_done = false;          // (set only between a sampling kernel and the decode step that follows it at once)
    record_history(m, m->ids.as<int>(), batch, 1, m->pos);
    try { decode_step(m, m->ids.as<int>(), batch); } catch (...) { m->prof = nullptr; throw; }
    m->prof = nullptr;
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    m->cur_batch = batch;
    int cnt = (int)prof.names.size();
    m->last_symbols = prof.symbols;
    *n = cnt;
    for (int i = 0; i < cnt && i < n_max; ++i) {
        float t = 0.0f;
        TSHIP_CHECK_HIP(hipEventElapsedTime(&t, prof.ev0[i], prof.ev1[i]));
        ms[i] = t;
        std::strncpy(names + (size_t)i * 48, prof.names[i].c_str(), 47);
        names[(size_t)i * 48 + 47] = 0;
    }
    TSHIP_END
}

TSHIP_API int TSHip_GptProfileSymbols(TSHipGpt* m, char* symbols, int stride, int n_max, int* n) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m && symbols && n && stride >= 2, "TSHip_GptProfileSymbols: bad argument");
    *n = (int)m->last_symbols.size();
    for (int i = 0; i < *n && i < n_max; ++i) {
        std::strncpy(symbols + (size_t)i * stride, m->last_symbols[i].c_str(), stride - 1);
        symbols[(size_t)i * stride + stride - 1] = 0;
    }
    TSHIP_END
}

TSHIP_API int TSHip_GptStepBytes(TSHipGpt* m, int batch, double* weight_bytes, double* kv_bytes) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(m && weight_bytes && kv_bytes, "TSHip_GptStepBytes: null argument");
    auto& c = m->c;
    const double s = (double)m->esz();
    const double h = c.hidden, Hd = (double)c.n_heads * m->D, Gd = (double)c.n_kv_heads * m->D, F = c.ffn_dim, V = c.vocab;
    double params = 0.0;
    for (int l = 0; l < c.n_layers; ++l) {
        params += h * Hd + 2.0 * h * Gd + Hd * h;
        if (m->L[l]->moe) params += h * c.n_experts + (double)std::min(c.n_experts, batch * c.experts_per_token) * 2.0 * h * 4.0 * h;
        else params += (m->gated ? 3.0 : 2.0) * h * F;
    }
    params += h * V;
    *weight_bytes = s * params + (double)batch * h * s;
    *kv_bytes = s * (double)c.n_layers * batch * Gd * 2.0 * (double)(m->pos + 1);
    TSHIP_END
}

}  // extern "C"
