/*
 * tship.h — C ABI of libtship.so, the native half of a TensorSharp.HIP backend for MI355X (gfx950).
 *
 * Conventions (the same ones the reference's GGML bridge uses between TensorSharp.GGML/GgmlNative.cs
 * and TensorSharp.GGML.Native/ggml_ops.cpp):
 *   - extern "C", cdecl, default visibility                              (ggml_ops.cpp:89-93, GgmlNative.cs:164)
 *   - every call returns int: 1 = success, 0 = failure                   (GgmlNative.cs:471-479)
 *   - on failure the message is kept per thread, read with TSHip_GetLastError()
 *                                                                        (ggml_ops.cpp:211-224, :4683-4686)
 *   - no C++ exception crosses the boundary                              (ggml_ops.cpp:4707-4722)
 *   - the caller owns every tensor buffer; the library keeps no tensor pointer after a call returns
 *   - calls are ordered on one library stream; functions that hand data to the host synchronise
 *   - any thread may call: a call holds the library's lock from entry to return, so calls from several threads
 *     (the reference issues ops from Parallel.For workers, BaseSeq2SeqFramework.cs:912-941) are serialised, each
 *     seeing its own last-error string; one TSHipGpt object is meant for one thread at a time, like a ggml context
 *
 * Tensor arguments are strided views (sizes and strides in ELEMENTS, outermost dimension first, exactly
 * TensorSharp.Tensor's Sizes/Strides, TensorSharp/Tensor.cs:12-125).  `data` is a DEVICE pointer already
 * advanced by StorageOffset.  Indices travel as float32 tensors, as everywhere in the reference
 * (Seq2SeqSharp/Applications/Decoder.cs:708-715).
 */
#ifndef TSHIP_H
#define TSHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TSHIP_API __attribute__((visibility("default")))
#define TSHIP_MAX_DIMS 6

/* TensorSharp/DType.cs:6-13 */
enum { TSHIP_F32 = 0, TSHIP_F16 = 1 };

typedef struct TSHipTensor {
    void*   data;                     /* device pointer (storage base + StorageOffset * element size) */
    int32_t dtype;                    /* TSHIP_F32 or TSHIP_F16 */
    int32_t ndim;                     /* 1..TSHIP_MAX_DIMS */
    int64_t sizes[TSHIP_MAX_DIMS];
    int64_t strides[TSHIP_MAX_DIMS];  /* in elements; 0 = expanded (broadcast) dimension */
} TSHipTensor;

/* ---- runtime: what HipAllocator / HipStorage need (TensorSharp/IAllocator.cs:13-20, Storage.cs:32-47,
 *      modelled on TensorSharp.CUDA/CudaStorage.cs:35-173: synchronous device<->host copies) ---- */
TSHIP_API const char* TSHip_GetLastError(void);                               /* cf. TSGgml_GetLastError */
TSHIP_API int TSHip_GetDeviceCount(int* count);
TSHIP_API int TSHip_Init(int device_id);                                      /* once per process; cf. ggml_ops.cpp:256-280 */
/* Device memory comes from a pool (cf. TensorSharp.CUDA/ContextState/PoolingDeviceAllocator.cs): freed blocks are cached
 * by size class and handed out again without a driver call or a device synchronisation (every use of a block is ordered
 * on the library stream).  TSHip_Free rejects pointers that TSHip_Malloc did not hand out. */
TSHIP_API int TSHip_Malloc(void** ptr, size_t bytes);                         /* IAllocator.Allocate */
TSHIP_API int TSHip_Free(void* ptr);                                          /* Storage.Destroy */
TSHIP_API int TSHip_PoolTrim(void);                                           /* give every cached block back to the driver */
/* number of hipMalloc calls the pool has made, bytes handed out, bytes cached for reuse (any pointer may be NULL) */
TSHIP_API int TSHip_GetPoolStats(size_t* device_allocations, size_t* bytes_in_use, size_t* bytes_cached);
TSHIP_API int TSHip_MemcpyH2D(void* dst, const void* src, size_t bytes);      /* Storage.CopyToStorage / SetElementsAsFloat */
TSHIP_API int TSHip_MemcpyD2H(void* dst, const void* src, size_t bytes);      /* Storage.CopyFromStorage / GetElementsAsFloat */
TSHIP_API int TSHip_MemcpyD2D(void* dst, const void* src, size_t bytes);
TSHIP_API int TSHip_Memset(void* dst, int value, size_t bytes);
TSHIP_API int TSHip_Synchronize(void);
TSHIP_API int TSHip_GetMemInfo(size_t* free_bytes, size_t* total_bytes);      /* IAllocator.GetAllocatedMemoryRatio */

/* ---- per-op surface: one entry per OpRegistry name the decode path issues (TensorSharp/Ops.cs:15-303).
 *      Signatures follow the CPU handlers in TensorSharp/Cpu/CpuBasicOps.cs; `result` is always supplied
 *      by the caller (the managed side allocates it with TensorResultBuilder.GetWriteTarget). ---- */

/* "copy" (Ops.cs:24-34, TensorApplyCPU.cs:282-306); also float2half / half2float when dtypes differ
 * (ComputeGraphTensor.cs:1427-1438, :1484-1495) */
TSHIP_API int TSHip_Copy(const TSHipTensor* result, const TSHipTensor* src);
/* "fill" */
TSHIP_API int TSHip_Fill(const TSHipTensor* result, float value);
/* "addmm": result = beta*src + alpha*m1*m2 (CpuBasicOps.cs:49-114) */
TSHIP_API int TSHip_Addmm(const TSHipTensor* result, float beta, const TSHipTensor* src, float alpha,
                          const TSHipTensor* m1, const TSHipTensor* m2);
/* "addmmbatch" (CpuBasicOps.cs:116-184) */
TSHIP_API int TSHip_AddmmBatch(const TSHipTensor* result, float beta, const TSHipTensor* src, float alpha,
                               const TSHipTensor* m1, const TSHipTensor* m2);
/* "indexselect": result[j,:] (+)= src[(int)indice[j],:], negative indices skipped (TensorApplyCPU.cs:1306-1333) */
TSHIP_API int TSHip_IndexSelect(const TSHipTensor* result, const TSHipTensor* src, const TSHipTensor* indice, int is_add);
/* "indexselectgrad": grad[(int)indice[j],:] += adj[j,:] in row order (TensorApplyCPU.cs:1336-1356) */
TSHIP_API int TSHip_IndexSelectGrad(const TSHipTensor* grad, const TSHipTensor* adj, const TSHipTensor* indice);
/* "rope" (CpuBasicOps.cs:1049-1066, TensorApplyCPU.cs:1148-1178): base 500000, adjacent pairs */
TSHIP_API int TSHip_RoPE(const TSHipTensor* result, const TSHipTensor* src, int seq_len, int row_offset);
/* same with the base as an argument (the reference has no such parameter) */
TSHIP_API int TSHip_RoPEEx(const TSHipTensor* result, const TSHipTensor* src, int seq_len, int row_offset, float base);
/* "rmsnorm" / "layernorm" (TensorApplyCPU.cs:1451-1496, :1360-1447); beta may be NULL */
TSHIP_API int TSHip_RMSNorm(const TSHipTensor* result, const TSHipTensor* src, const TSHipTensor* gamma,
                            const TSHipTensor* beta, float eps);
TSHIP_API int TSHip_LayerNorm(const TSHipTensor* result, const TSHipTensor* src, const TSHipTensor* gamma,
                              const TSHipTensor* beta, float eps);
/* "softmax" over the last dimension (TensorApplyCPU.cs:1230-1268) */
TSHIP_API int TSHip_Softmax(const TSHipTensor* result, const TSHipTensor* src);
/* "argmax" along `dim`, float indices, first maximum wins (TensorApplyCPU.cs:339-360) */
TSHIP_API int TSHip_Argmax(const TSHipTensor* result, const TSHipTensor* src, int dim);
/* "topK": descending values + float indices with the reference's insertion rule (TensorApplyCPU.cs:1099-1146) */
TSHIP_API int TSHip_TopK(const TSHipTensor* out_val, const TSHipTensor* out_idx, const TSHipTensor* src, int k);

/* element-wise families (TensorApplyCPU.cs:378-673, :852-861, :1747-1801) */
enum { TSHIP_ADD = 0, TSHIP_SUB = 1, TSHIP_MUL = 2, TSHIP_DIV = 3 };
enum { TSHIP_RELU = 0, TSHIP_SILU = 1, TSHIP_LEAKYRELU = 2, TSHIP_EXP = 3, TSHIP_LOG = 4, TSHIP_NEG = 5,
       TSHIP_SIGMOID = 6, TSHIP_TANH = 7, TSHIP_SQRT = 8, TSHIP_ABS = 9 };
/* "addt" "subt" "mult" "divt": result = lhs op rhs (rhs may be an expanded view) */
TSHIP_API int TSHip_BinaryTensor(int op, const TSHipTensor* result, const TSHipTensor* lhs, const TSHipTensor* rhs);
/* "addv" "subv" "mulv" "divv": result = src op scalar */
TSHIP_API int TSHip_BinaryScalar(int op, const TSHipTensor* result, const TSHipTensor* src, float scalar);
/* "relu" "SiLU" "LeakyReLU" "exp" "log" "neg" "sigmoid" "tanh" "sqrt" "abs" */
TSHIP_API int TSHip_Unary(int op, const TSHipTensor* result, const TSHipTensor* src);
/* "buildtrimask" / "buildselftrimask" (TensorApplyCPU.cs:1016-1065) */
TSHIP_API int TSHip_BuildTriMask(const TSHipTensor* result, float value, float masked_value);
TSHIP_API int TSHip_BuildSelfTriMask(const TSHipTensor* result, const TSHipTensor* original_lengths,
                                     int padded_seq_len, float value, float masked_value);
/* "gather": result[.., j, ..] = src[.., (long)indices[.., j, ..], ..] along `dim`; "scatter_fill": result[.., (long)indices[..], ..] =
 * value (CpuIndexingOps.cs:23-56, :141-167; TensorApplyCPU.cs:200-257).  The beam search loop issues them on the probabilities
 * (Decoder.cs:766, :788).  An index outside the dimension fails the call. */
TSHIP_API int TSHip_Gather(const TSHipTensor* result, const TSHipTensor* src, int dim, const TSHipTensor* indices);
TSHIP_API int TSHip_ScatterFill(const TSHipTensor* result, float value, int dim, const TSHipTensor* indices);
/* "iscorrupted": *corrupted = 1 if any element is not finite (TensorApplyCPU.cs:1212-1228) */
TSHIP_API int TSHip_IsCorrupted(const TSHipTensor* src, int* corrupted);

/* Top-p sampling on the device, one row per sequence; semantics of ComputeGraphTensor.TopPSample
 * (Seq2SeqSharp/Tools/ComputeGraphTensor.cs:2305-2403) with the random draw of row i replaced by uniforms[i].
 * probs [rows, K] f32, uniforms [rows] f32, result [rows,1] f32 (float indices).
 * TSHip_TopPSample: decodedSequences = null (no decay).
 * TSHip_TopPSampleEx: decodedSequences given as host_seqs [rows][seq_ld] int32 with host_seq_lens [rows]; a token that
 * occurs in its row's sequence is decayed by pow(dist / len, repeat_penalty) (:2320-2345; the reference's default is 2). */
TSHIP_API int TSHip_TopPSample(const TSHipTensor* result, const TSHipTensor* probs, const TSHipTensor* uniforms, float top_p);
TSHIP_API int TSHip_TopPSampleEx(const TSHipTensor* result, const TSHipTensor* probs, const TSHipTensor* uniforms, float top_p, float repeat_penalty,
                                 const int32_t* host_seqs, const int32_t* host_seq_lens, int seq_ld);

/* TSHip_TopPSample for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): no counterpart in the reference.  Same arguments, same kernels and same result as
 * TSHip_TopPSample, but the pipeline's scratch (sort keys, indices, running sums, digit counts) lives in a fixed 6 MiB
 * device array inside the library instead of a per-call allocation, and nothing is allocated, freed or synchronised.
 * Limit: rows * 20 * round_up(columns, 64) + rows * ceil(columns / 1024) * 1024 bytes must fit in 6 MiB (about 300000
 * probabilities, e.g. 8 rows of 32000); larger inputs fail with an error.  TSHip_Init must have been called.  All calls
 * on a GPU share that GPU's array: calls that overlap in time on one GPU race; calls on the library stream do not. */
TSHIP_API int TSHip_TopPSampleNoAlloc(const TSHipTensor* result, const TSHipTensor* probs, const TSHipTensor* uniforms, float top_p);

/* ---- fused GPTDecoder path: one object per model replica, preallocated compact KV cache, the whole
 *      token loop on the device (replaces GPT.RunForwardOnSingleDevice, Seq2SeqSharp/Applications/GPT.cs:212-335,
 *      Decoder.GPTDecode, Applications/Decoder.cs:648-794, and GPTDecoder.Decode, Networks/GPTDecoder.cs:153-191). ---- */
typedef struct TSHipGptConfig {
    int32_t n_layers, hidden, n_heads, n_kv_heads, ffn_dim, vocab;
    int32_t attn_type;          /* 0 = MultiHeadAttention (fused QKV [h,3h], columns ordered [3][H][d]), 1 = GroupQueryAttention */
    int32_t norm_type;          /* 0 = RMSNorm, 1 = LayerNorm */
    int32_t act;                /* 0 ReLU, 1 SiLU, 2 LeakyReLU, 3 "SwiGLU" as the reference computes it (no SiLU on the gate),
                                   4 = gated with SiLU (not a reference mode) */
    int32_t n_experts;          /* > 1: layers 2.. use MoEFeedForward (Networks/GPTDecoder.cs:114-124) */
    int32_t experts_per_token;
    float   norm_eps;
    float   rope_base;          /* the reference's literal is 500000 */
    int32_t use_rope;
    int32_t dtype;              /* TSHIP_F32 or TSHIP_F16: storage type of weights and KV cache */
    int32_t max_batch;
    int32_t max_seq_len;        /* KV cache capacity per sequence (prompt + generated) */
    /* Segment embeddings (IModel.EnableSegmentEmbeddings / MaxSegmentNum; table "SegmentEmbedding" [max_segments, hidden] built by
     * Misc.CreateAuxEmbeddings, Utils/Misc.cs:164-168): 0 = none.  TensorUtils.CreateTokensEmbeddings (Utils/TensorUtils.cs:60-72,
     * 147-152) adds row s of the table to the scaled embedding of a token, s = number of sep_token_id tokens ("[SEP]",
     * SENTTAGS.SEP = 3 in the reference's vocabularies) that come BEFORE it in the token list of the call: a prefill counts
     * through its own tokens from 0, and a cached decode step feeds one token per sequence, which therefore always gets
     * segment 0 (Applications/Decoder.cs:661-673).  This library counts the same way. */
    int32_t max_segments;
    int32_t sep_token_id;
} TSHipGptConfig;

typedef struct TSHipGpt TSHipGpt;

TSHIP_API int TSHip_GptCreate(const TSHipGptConfig* cfg, TSHipGpt** out);
TSHIP_API int TSHip_GptDestroy(TSHipGpt* m);
/* weights by the reference's saved parameter names, from host float32 arrays, shape as saved
 * (WeightTensor.SetWeightArray, Seq2SeqSharp/Tools/WeightTensor.cs:504-520); converted to the model dtype
 * with round-to-nearest-even (BasicTypesStructAsTypes.cs:800-840) */
TSHIP_API int TSHip_GptSetWeight(TSHipGpt* m, const char* name, const float* host_data, int ndim, const int64_t* sizes);
/* call once after the last TSHip_GptSetWeight: checks that every parameter is present */
TSHIP_API int TSHip_GptFinalize(TSHipGpt* m);
/* drop the KV cache contents (GPT.cs:236-247: a new dictionary per call) */
TSHIP_API int TSHip_GptReset(TSHipGpt* m);
/* prefill: ids [batch, prompt_len] int32 on the host, equal lengths; appends them to the cached sequences (the cache is
 * empty after Create / Reset; a later call continues the same sequences, e.g. the next turn of a dialogue whose cache
 * was kept, GPT.cs:236-247,312-328) and leaves the last-position logits on the device (Decoder.cs:679-716) */
TSHIP_API int TSHip_GptPrefill(TSHipGpt* m, const int32_t* host_ids, int batch, int prompt_len);
/* prefill of sequences of different lengths, as the reference runs them when padding is allowed (Decoder.cs:656, 687-690):
 * ids [batch, padded_len] hold every sequence padded with the END tag to the longest (BuildInTokens.PadSentences,
 * Corpus/BuildInTokens.cs:68-101), host_lens [batch] the original lengths.  Masking is BuildSelfTriMask's
 * (TensorApplyCPU.cs:1040-1065): a row inside its sequence sees the columns up to itself, a padding row has every column
 * masked (so it attends to the whole padded sequence).  As in the reference, all sequences continue from position
 * padded_len: the logits are those of every row's LAST PADDED position and the padding stays in the cache.  The cache must
 * be empty (Create / Reset). */
TSHIP_API int TSHip_GptPrefillPadded(TSHipGpt* m, const int32_t* host_ids, const int32_t* host_lens, int batch, int padded_len);
/* one decode step with the given tokens (Decoder.cs:661-678); leaves logits on the device */
TSHIP_API int TSHip_GptDecode(TSHipGpt* m, const int32_t* host_ids, int batch);
/* DecodingOptions.RepeatPenalty (Applications/DecodingOptions.cs:23, default 2.0 there; 0 here until set): top-p sampling
 * decays tokens that already occur in the sequence, prompt included (Decoder.cs:761).  A non-zero value makes the model
 * keep the last position of every token per sequence, from the next prompt on: set it before TSHip_GptPrefill (or after
 * TSHip_GptReset).  TSHip_GptSetKV / TSHip_GptSetSeqLen do not reconstruct that history.  Greedy decoding ignores it. */
TSHIP_API int TSHip_GptSetRepeatPenalty(TSHipGpt* m, float repeat_penalty);
/* DecodingOptions.BlockedTokens (Decoder.cs:745-753: -1 is added to their probabilities before the choice): the tokens
 * are never chosen, by argmax or by top-p.  n = 0 clears the list. */
TSHIP_API int TSHip_GptSetBlockedTokens(TSHipGpt* m, const int32_t* ids, int n);
/* sampling modes */
enum { TSHIP_GREEDY = 0, TSHIP_TOPP = 1 };
/* choose next tokens from the logits on the device: softmax (after division by temperature when
 * sampling and temperature != 1, Decoder.cs:720-732) then argmax or top-p; uniforms: host [batch] (top-p only) */
TSHIP_API int TSHip_GptSample(TSHipGpt* m, int mode, float top_p, float temperature, const float* host_uniforms, int32_t* host_ids_out);
/* n_steps of (sample from current logits -> decode the sampled tokens), all on the device; only token ids come
 * back: host_ids_out [n_steps, batch].  host_uniforms [n_steps, batch] for top-p (else NULL).
 * elapsed_ms (optional): device time of the loop measured with events on the library stream. */
TSHIP_API int TSHip_GptGenerate(TSHipGpt* m, int n_steps, int mode, float top_p, float temperature,
                                const float* host_uniforms, int32_t* host_ids_out, float* elapsed_ms);
/* the same loop with the reference's stop rule (GPT.cs:299-302, Decoder.AreAllSentsCompleted, Decoder.cs:207-221): stops
 * after the first step at which every sequence's new token is eos_id (the vocabulary's END tag, 0 in the reference).
 * *steps_done steps were run; host_ids_out [max_steps, batch] holds that many rows.  The host looks at every step's
 * tokens, which costs one small copy and one synchronisation per step. */
TSHIP_API int TSHip_GptGenerateUntil(TSHipGpt* m, int max_steps, int eos_id, int mode, float top_p, float temperature,
                                     const float* host_uniforms, int32_t* host_ids_out, int* steps_done, float* elapsed_ms);
/* ---- beam search (Decoder.cs:756-792, GPT.cs:264-297, Utils/BeamSearch.cs:36-46).  Hypotheses are rows of the cached batch. ----
 * TSHip_GptBeamPick: from the logits on the device, n_picks picks per row as the reference makes them: probabilities =
 * softmax (after the division by the temperature when sampling), pick = Argmax (greedy) or TopPSample (with the repeat
 * penalty and the blocked tokens set on the model; host_uniforms [n_picks, batch]), ScatterFill(probs, 0) at the picked
 * index before the next pick.  host_ids_out [n_picks, batch]; host_logp_out [n_picks, batch] = log of the picked
 * probability (the reference adds its negative to the hypothesis' score).  Nothing is appended to the sequences. */
TSHIP_API int TSHip_GptBeamPick(TSHipGpt* m, int n_picks, int mode, float top_p, float temperature, const float* host_uniforms,
                                int32_t* host_ids_out, float* host_logp_out);
/* Gather the cached sequences: row i of the new batch continues old row host_src_rows[i] (rows may repeat: a hypothesis
 * with several surviving children; new_batch may differ from the old batch, at most max_batch).  KV cache and token
 * history move; the logits on the device are stale until the next TSHip_GptDecode. */
TSHIP_API int TSHip_GptReorderRows(TSHipGpt* m, const int32_t* host_src_rows, int new_batch);
/* BeamSearch.GetTopNBSS: indices of the top_n lowest scores among scores[0..n), in the order the reference's
 * FixedSizePriorityQueue enumerates them (AdvUtils/FixedSizePriorityQueue.cs; not sorted).  kept: top_n entries. */
TSHIP_API int TSHip_BeamTopN(const float* scores, int n, int top_n, int32_t* kept, int* n_kept);

/* inspection for parity tests */
TSHIP_API int TSHip_GptGetLogits(TSHipGpt* m, float* host_out /* [batch, vocab] */);
TSHIP_API int TSHip_GptGetHidden(TSHipGpt* m, float* host_out /* [batch, hidden], after the final norm */);
TSHIP_API int TSHip_GptGetSeqLen(TSHipGpt* m, int* len);
/* KV cache rows of one layer as float32: which = 0 keys (after RoPE), 1 values; layout [batch, n_kv_heads, len, head_dim] */
TSHIP_API int TSHip_GptGetKV(TSHipGpt* m, int layer, int which, float* host_out);
/* install cache contents (same layout) and the sequence length: lets a benchmark start at a given context length */
TSHIP_API int TSHip_GptSetKV(TSHipGpt* m, int layer, int which, const float* host_in, int batch, int len);
TSHIP_API int TSHip_GptSetSeqLen(TSHipGpt* m, int batch, int len);

/* Saved sequence sets, device to device.  The reference parks the KV tensors of a finished request in a MemoryCache keyed by
 * the generated text (sliding expiry of ten minutes) and takes them out again when a later request continues that text
 * (Seq2SeqSharp/Applications/GPT.cs:153-173, 236-247, 312-328); several conversations are parked at a time.  Here
 * TSHip_GptSaveRows copies the used prefix of every layer's cache regions of the current sequences (in the cache's own
 * layout and type: no host round trip, no float32 expansion), the logits of the last step and the token history into a
 * snapshot that lives in device memory until TSHip_GptFreeSnapshot; TSHip_GptRestoreRows puts a snapshot back as the
 * model's current sequences (rows 0 .. batch-1, length as saved), after which TSHip_GptSample / TSHip_GptDecode /
 * TSHip_GptPrefill (append) continue bit for bit as if nothing had run in between.  The model may serve other sequences
 * between the two calls; the dictionary keyed by text, and its expiry, belong to the caller (HipGptDecoder.cs).  A snapshot
 * fits any model object of the same shape and type whose cache is long enough. */
typedef struct TSHipGptSnapshot TSHipGptSnapshot;
TSHIP_API int TSHip_GptSaveRows(TSHipGpt* m, TSHipGptSnapshot** out);
TSHIP_API int TSHip_GptRestoreRows(TSHipGpt* m, const TSHipGptSnapshot* snapshot);
TSHIP_API int TSHip_GptSnapshotInfo(const TSHipGptSnapshot* snapshot, int* batch, int* len, int64_t* device_bytes);
TSHIP_API int TSHip_GptFreeSnapshot(TSHipGptSnapshot* snapshot);
/* routing of MoE layer `layer` at the last step: top_idx/top_val [rows, k], probs [rows, E] (host, float32) */
TSHIP_API int TSHip_GptGetMoeRouting(TSHipGpt* m, int layer, float* top_idx, float* top_val, float* probs);
/* per-kernel device times of one decode step (events around every launch on the library stream).
 * names: buffer of n_max entries of 48 chars; ms: n_max floats; *n receives the number of launches. */
TSHIP_API int TSHip_GptProfileDecode(TSHipGpt* m, const int32_t* host_ids, int batch, char* names, float* ms, int n_max, int* n);
/* the launched kernel symbols (demangled, as a profiler's kernel trace names them) of the step TSHip_GptProfileDecode timed
 * last, in launch order: n_max entries of `stride` chars */
TSHIP_API int TSHip_GptProfileSymbols(TSHipGpt* m, char* symbols, int stride, int n_max, int* n);
/* algorithmic bytes one decode step moves at the current sequence length (weights once, compact KV once) */
TSHIP_API int TSHip_GptStepBytes(TSHipGpt* m, int batch, double* weight_bytes, double* kv_bytes);


/* Environment switches (test hooks, read once at the start of every TSHip_GptPrefill*, TSHip_GptDecode,
 * TSHip_GptGenerate*, TSHip_GptProfileDecode call; a value outside the listed ones makes the call fail).  None of them
 * changes results beyond what the tests that use them state; production runs set none.
 *   TSHIP_NO_GRAPH=1          the generate loop launches its kernels one by one instead of replaying a captured HIP graph
 *   TSHIP_ATTN_SPLITS=n       decode attention: n blocks per (sequence, KV head) pair (default: chosen from the batch and context)
 *   TSHIP_FFN_TILES=10|15|20|30|40   decode FFN up projection: column tiles per block x 10 (15 = a tile and a half)
 *   TSHIP_PATCH_ROWS=1|2|4|8  prefill GEMM: row tiles per tile patch of an XCD
 *   TSHIP_ATTN_NQ=1|2         prefill attention: groups of 16 MFMA columns per wavefront
 *   TSHIP_NO_KV_FUSE=1        prefill: the QKV projection leaves the cache write to a kernel of its own
 *   TSHIP_NO_MOE_BATCH=1      prefill of MoE layers: the experts' row counts are read back, the rows gathered and one GEMM
 *                             launched per expert, instead of one launch per projection with everything on the device */

#ifdef __cplusplus
}
#endif
#endif /* TSHIP_H */
