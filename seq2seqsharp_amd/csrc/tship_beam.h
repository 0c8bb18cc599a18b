// Beam search primitives of the fused GPTDecoder path.  Included by tship_gpt.hip after the model object is defined.
//
// The reference's beam search (Seq2SeqSharp/Applications/Decoder.cs:756-792, Applications/GPT.cs:264-297,
// Utils/BeamSearch.cs:36-46) keeps BeamSearchSize hypotheses per sequence: every step it makes BeamSearchSize picks from
// the probabilities of every hypothesis (a pick, then ScatterFill(probs, 0) at the picked index, then the next pick),
// adds -log p of each pick to the hypothesis' score, and keeps the BeamSearchSize lowest scores per sequence.  It runs
// that without a KV cache (GPT.cs:238-241: the cache dictionary only exists for BeamSearchSize == 1) and recomputes every
// hypothesis from its first token at every step.  Here the hypotheses are rows of the one cached batch: the picks run on
// the device (TSHip_GptBeamPick), the host prunes (TSHip_BeamTopN restates the reference's queue) and the surviving
// hypotheses' cache rows are gathered into place (TSHip_GptReorderRows) before the chosen tokens are decoded.
#pragma once

namespace tship {

// probabilities of every row of logits: (float)exp(x - max) / sum (TensorApplyCPU.cs:1230-1268), after the division by the
// temperature when sampling (Decoder.cs:720-723).  grid (rows), 1024 threads.
__global__ __launch_bounds__(1024) void beam_probs_kernel(const float* __restrict__ logits, long ld, int V, float temperature, int divide,
                                                          float* __restrict__ probs, long ldp) {
    __shared__ float sred[16];
    const int r = blockIdx.x, t = threadIdx.x;
    const float* row = logits + (long)r * ld;
    float mx = -INFINITY;
    for (int i = t; i < V; i += 1024) { const float x = divide ? row[i] / temperature : row[i]; mx = fmaxf(mx, x); }
    mx = wave_max(mx);
    if ((t & 63) == 0) sred[t >> 6] = mx;
    __syncthreads();
    mx = sred[0];
#pragma unroll
    for (int w = 1; w < 16; ++w) mx = fmaxf(mx, sred[w]);
    __syncthreads();
    float sum = 0.0f;
    for (int i = t; i < V; i += 1024) { const float x = divide ? row[i] / temperature : row[i]; sum += expf(x - mx); }
    sum = wave_sum(sum);
    if ((t & 63) == 0) sred[t >> 6] = sum;
    __syncthreads();
    sum = sred[0];
#pragma unroll
    for (int w = 1; w < 16; ++w) sum += sred[w];
    for (int i = t; i < V; i += 1024) { const float x = divide ? row[i] / temperature : row[i]; probs[(long)r * ldp + i] = expf(x - mx) / sum; }
}

// after a pick: Gather + Log of the picked probability (Decoder.cs:766-767), then ScatterFill(probs, 0) at the picked index
// (Decoder.cs:788): one thread per row
__global__ void beam_take_kernel(float* __restrict__ probs, long ldp, const int* __restrict__ ids, int rows, int* __restrict__ ids_out,
                                 float* __restrict__ logp_out) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= rows) return;
    const int id = ids[r];
    ids_out[r] = id;
    logp_out[r] = logf(probs[(long)r * ldp + id]);
    probs[(long)r * ldp + id] = 0.0f;
}

// rows of a [rows][row_stride] table gathered into a dense temporary and back: dst row i = old row src[i].  Only the first
// `used` bytes of every `chunk`-byte piece of a row are live (the cached positions of one KV head).
// grid (pieces per row, new_rows), 256 threads, 16 bytes per thread and round
__global__ __launch_bounds__(256) void rows_gather_kernel(const char* __restrict__ table, long row_stride, long chunk, long used, const int* __restrict__ src,
                                                          char* __restrict__ tmp, int to_tmp) {
    const long piece = blockIdx.x; const int i = blockIdx.y;
    const long off = piece * chunk;
    const char* from = to_tmp ? table + (long)src[i] * row_stride + off : tmp + (long)i * row_stride + off;
    char* to = to_tmp ? tmp + (long)i * row_stride + off : (char*)table + (long)i * row_stride + off;
    for (long b = (long)threadIdx.x * 16; b < used; b += 256 * 16) *(uint4*)(to + b) = *(const uint4*)(from + b);
}

// BeamSearch.GetTopNBSS (Utils/BeamSearch.cs:36-46): a FixedSizePriorityQueue (AdvUtils/FixedSizePriorityQueue.cs) with
// ComparableItemComparer(false) (Tools/ComparableItem.cs:31-50), every candidate enqueued in order, then enumerated.
// The queue keeps two array heaps: `top` holds the better half (lower scores) with its best element at the root, `bottom`
// the other half with its worst at the root; a full queue replaces bottom's root when the newcomer is better.
// Enumeration is top in array order followed by bottom in reverse array order, which is the order the surviving
// hypotheses take.
class TopNQueue {
public:
    explicit TopNQueue(int capacity) : cap_(capacity), count_(0), bottom_size_(0), top_size_(0) {
        const int bottom_cap = std::max(capacity / 2, 1), top_cap = std::max(capacity - bottom_cap, 1);
        top_.resize(top_cap); bottom_.resize(bottom_cap);
    }
    struct Item { float score; int index; };
    bool enqueue(Item t) {
        if (cap_ == count_) {
            if (cap_ == 1) { if (!better(t, top_[0], true)) return false; top_[0] = t; return true; }
            if (!better(t, bottom_[0], true)) return false;
            bottom_[0] = t;
            const int updated = down_heapify(bottom_, 0, bottom_size_, false);
            if (!semi_leaf(updated, bottom_size_)) return true;
            const int it = check_boundary_upwards(updated);
            if (it == -1) return true;
            up_heapify(top_, it, true);
            return true;
        }
        ++count_;
        if (bottom_size_ < top_size_) {
            const int pos = bottom_size_++;
            bottom_[pos] = t;
            const int up = check_boundary_upwards(pos);
            if (up == -1) up_heapify(bottom_, pos, false); else up_heapify(top_, up, true);
            return true;
        }
        const int pos = top_size_++;
        top_[pos] = t;
        const int bt = check_boundary_downwards(pos);
        if (bt == -1) up_heapify(top_, pos, true); else up_heapify(bottom_, bt, false);
        return true;
    }
    std::vector<Item> enumerate() const {
        std::vector<Item> out;
        for (int i = 0; i < top_size_; ++i) out.push_back(top_[i]);
        for (int i = bottom_size_ - 1; i >= 0; --i) out.push_back(bottom_[i]);
        return out;
    }
private:
    // ComparableItemComparer(false).Compare(x, y) = -sign(x.Score - y.Score); Better(t1, t2, fTop) = fTop ? cmp > 0 : cmp < 0
    static int sign(float v) { return v > 0.0f ? 1 : (v < 0.0f ? -1 : 0); }      // (Math.Sign; a NaN score throws there, it cannot occur here)
    static bool better(const Item& a, const Item& b, bool f_top) { const int c = -sign(a.score - b.score); return f_top ? c > 0 : c < 0; }
    static int parent(int i) { return (i - 1) / 2; }
    static int left(int i) { return 2 * i + 1; }
    static int right(int i) { return 2 * i + 2; }
    static bool semi_leaf(int i, int size) { return right(i) >= size; }
    int bottom_node(int i) const { if (i < bottom_size_) return i; return i % 2 == 1 ? parent(i) : i - 1; }
    int top_node1(int i) const { if (left(i) >= bottom_size_ && left(i) < top_size_) return left(i); return i; }
    int top_node2(int i) const {
        if (i == bottom_size_ - 1 && i % 2 == 1 && top_size_ > bottom_size_) return i + 1;
        if (left(i) >= bottom_size_ && left(i) < top_size_) return left(i);
        return i;
    }
    static int up_heapify(std::vector<Item>& a, int i, bool f_top) {
        while (i > 0) { const int p = parent(i); if (!better(a[i], a[p], f_top)) return i; std::swap(a[i], a[p]); i = p; }
        return i;
    }
    static int down_heapify(std::vector<Item>& a, int i, int size, bool f_top) {
        for (;;) {
            const int l = left(i), r = right(i); int best = i;
            if (l < size && better(a[l], a[best], f_top)) best = l;
            if (r < size && better(a[r], a[best], f_top)) best = r;
            if (best == i) return i;
            std::swap(a[i], a[best]); i = best;
        }
    }
    int check_boundary_upwards(int bpos) {
        const int t1 = top_node1(bpos), t2 = top_node2(bpos); int b = -1;
        if (better(bottom_[bpos], top_[t1], true)) b = t1;
        if (better(bottom_[bpos], top_[t2], true) && (b == -1 || better(top_[t1], top_[t2], true))) b = t2;
        if (b == -1) return -1;
        std::swap(top_[b], bottom_[bpos]);
        return b;
    }
    int check_boundary_downwards(int tpos) {
        const int bpos = bottom_node(tpos);
        if (bpos == -1) return -1;
        if (bpos >= bottom_size_ || !better(bottom_[bpos], top_[tpos], true)) return -1;
        std::swap(top_[tpos], bottom_[bpos]);
        return bpos;
    }
    int cap_, count_, bottom_size_, top_size_;
    std::vector<Item> top_, bottom_;
};

}  // namespace tship
