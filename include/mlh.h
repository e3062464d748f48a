/*
 * mlh.h -- C ABI of the MI355X (gfx950) device layer for the mini-llm inference
 * token loop.  This is the only interface through which host code reaches HIP:
 * plain pointers and sizes, int status codes (0 = ok, < 0 = error; text from
 * mlh_last_error), no C++ or torch types.
 *
 * Each entry point names the reference interface it replaces (file:line in
 * daniel-chermetz/mini-llm-cuda).  The reference keeps all of this in process
 * globals (network_globals.h:136-241); here one mlh_ctx owns every device
 * allocation, one HIP stream and the captured decode graphs.  A context is not
 * thread-safe; different contexts are independent.
 */
#ifndef MLH_H
#define MLH_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MLH_MAX_LAYERS 64

#define MLH_KIND_ATTENTION 0 /* softmax attention block (inference.cu:401-610) */
#define MLH_KIND_GDN 1       /* gated-delta-net block (no reference counterpart) */

#define MLH_DTYPE_F32 0
#define MLH_DTYPE_BF16 1 /* matrices rounded to bf16 (RNE) at upload, fp32 accumulate */

/* Runtime form of the compile-time macros of network_meta.h:3-20 (same names),
 * plus the fields the reference does not have. */
typedef struct {
    int32_t dim;
    int32_t attnHeads;
    int32_t headDim; /* attnHeads * headDim must equal dim (inference.cu:511-573 splits dim by head) */
    int32_t ffnDim;
    int32_t transformers;
    int32_t maxL;
    int32_t vocabSize;
    float ropeDenomBase;
    int32_t qkRmsNorm;   /* CONFIG_QK_RMS_NORM,  attention layers only */
    int32_t queryGating; /* CONFIG_QUERY_GATING, attention layers only */
    int32_t gdnHeads, gdnDk, gdnDv;
    int32_t pleDim;      /* per-layer-embedding width, 0 = none */
    int32_t weightDtype; /* MLH_DTYPE_* */
    int32_t maxSeqs;     /* concurrent sequences held on the device (>= 1) */
    int32_t layerKinds[MLH_MAX_LAYERS]; /* by FILE index: block 0 is the top of the stack (inference.cu:384-385) */
} mlh_hparams;

/* Tensor ids.  Per-layer ids follow the read order of load_model.cu:411-450;
 * the tail (GDN gates, per-layer embeddings) extends it. */
enum {
    MLH_T_TOKEN_EMBEDDINGS = 0, /* [vocabSize, dim]   embedding_weights (network_globals.h:150-151) */
    MLH_T_FINAL_RMS_GAMMA = 1,  /* [dim]              final_rms_weights */
    MLH_T_RMS_GAMMA = 2,        /* [dim]              rms1_weights */
    MLH_T_QUERY = 3,            /* [dim or Hg*dk, dim] query_weights */
    MLH_T_KEY = 4,              /*                    key_weights */
    MLH_T_VALUE = 5,            /* [dim or Hg*dv, dim] value_weights */
    MLH_T_OUTPUT_PROJ = 6,      /* [dim, dim or Hg*dv] output_proj_weights */
    MLH_T_RMS_GAMMA2 = 7,       /* [dim]              rms2_weights */
    MLH_T_FFN_1A = 8,           /* [ffnDim, dim]      ffn_right_1_weights (gate, SiLU branch) */
    MLH_T_FFN_1B = 9,           /* [ffnDim, dim]      ffn_right_2_weights (up) */
    MLH_T_FFN_2 = 10,           /* [dim, ffnDim]      ffn_left_weights (down) */
    MLH_T_QUERY_RMS_GAMMA = 11, /* [dim]              query_RMS_weights */
    MLH_T_KEY_RMS_GAMMA = 12,   /* [dim]              key_RMS_weights */
    MLH_T_GATED_QUERY = 13,     /* [dim, dim]         gated_query_weights */
    MLH_T_GDN_ALPHA_W = 14,     /* [gdnHeads, dim] */
    MLH_T_GDN_ALPHA_B = 15,     /* [gdnHeads] */
    MLH_T_GDN_BETA_W = 16,      /* [gdnHeads, dim] */
    MLH_T_GDN_BETA_B = 17,      /* [gdnHeads] */
    MLH_T_PLE_TABLE = 18,       /* [vocabSize, pleDim] */
    MLH_T_PLE_GATE = 19,        /* [pleDim, dim] */
    MLH_T_PLE_UP = 20,          /* [dim, pleDim] */
    MLH_T_COUNT = 21
};

typedef struct mlh_ctx mlh_ctx;

/* Last error text of a context (ctx == NULL: of the last failed mlh_create or context-free call on this thread). */
const char* mlh_last_error(const mlh_ctx* ctx);

/* Number of visible HIP devices (0 when there is none; never fails). */
int mlh_device_count(void);

/* Replaces allocateMemory(true) (memory_allocation.cu:326-557): validates the
 * hyper-parameters, allocates weights, KV pages, GDN states and scratch on
 * device `device`, creates the stream.  Weights start zeroed. */
int mlh_create(const mlh_hparams* hp, int device, mlh_ctx** out);
void mlh_destroy(mlh_ctx* ctx);

/* Replaces the cudaMemcpy of each tensor in loadModel (load_model.cu:366-372,
 * 383-388,429-434,456-461).  `host` is fp32, row-major [rows, cols] exactly as
 * stored in model.bin ([out, in]; the reference transposes to column-major for
 * cuBLAS, this layer consumes the file order directly).  layer is the FILE
 * block index, ignored for the two global tensors.  1-D tensors: cols = 1. */
int mlh_upload_tensor(mlh_ctx* ctx, int layer, int tensor_id, const float* host, int rows, int cols);

/* Replaces the RoPE table upload of memory_allocation.cu:383-388.  tab is the
 * host table of getPreComputedRopeTheta (inference.cu:364-374): [maxL, headDim]. */
int mlh_upload_rope_table(mlh_ctx* ctx, const float* tab, int n);

/* Must be called once after the uploads and before any forward call: checks
 * that every tensor the hyper-parameters require has arrived. */
int mlh_finalize(mlh_ctx* ctx);

/* Empties a sequence (length 0, GDN states zero).  seq = -1: all sequences.
 * The reference has one implicit sequence in seqTokenIndices (network_globals.h:147-148). */
int mlh_reset(mlh_ctx* ctx, int seq);
int mlh_seq_len(mlh_ctx* ctx, int seq);
int mlh_max_len(const mlh_ctx* ctx);    /* maxL of the context */
int mlh_vocab_size(const mlh_ctx* ctx); /* vocabSize of the context */

/* KV pages: every attention layer keeps K and V in pages of mlh_kv_page_size()
 * positions; sequence s, page j lives in pool slot table[s*pagesPerSeq + j].
 * The default table is the identity.  Replaces nothing in the reference (it has
 * no cache, inference_orchestrator.cu:64-65). */
int mlh_kv_page_size(void);
int mlh_set_page_table(mlh_ctx* ctx, const int32_t* table, int n);

/* Appends n tokens to sequence seq and leaves the logits of the last one
 * readable.  Together with mlh_decode_step this replaces runInference(L)
 * (inference.cu:376-751) as used by the token loop: the reference recomputes
 * all L columns per token, here positions already in the cache are not redone. */
int mlh_prefill(mlh_ctx* ctx, int seq, const int32_t* ids, int n);

/* The same for nseg distinct sequences in one pass: segment s appends lens[s]
 * tokens (ids holds the segments back to back) to sequence seqs[s].  With 16
 * or more tokens in the call, every projection is one MFMA GEMM over all
 * tokens (cuBLAS SGEMM over the L columns in the reference, inference.cu:409-449,
 * 575-596, 634-699), attention is tiled and causal over the pages
 * (inference.cu:511-573), GDN layers run their recurrence over the segment. */
int mlh_prefill_batch(mlh_ctx* ctx, int nseg, const int32_t* seqs, const int32_t* ids, const int32_t* lens);

/* Teacher-forced forward: appends n tokens to seq like mlh_prefill and returns what
 * runInference(L) leaves on the device for ALL L columns: logits_out and probs_out are
 * [n, vocabSize] (position-major, the reference's column-major [V x L] buffers
 * vocabScores_DEVICE / vocabScores_postSoftmax_DEVICE, inference.cu:723-749); either may be
 * null.  mean_nll (may be null) receives the mean over positions 0..n-2 of
 * -log max(p(ids[i+1] | ids[0..i]), 1e-4), the sequence loss processSequence prints
 * (training_orchestrator.cu:289-359, clamp at :343-347).  Allocates its own staging buffers per call. */
int mlh_forward_full(mlh_ctx* ctx, int seq, const int32_t* ids, int n, float* logits_out, float* probs_out, float* mean_nll);

/* 0 (default): GEMM prefill when the call has 16 or more tokens and dim, ffnDim,
 * pleDim and the mixing widths are multiples of 32 (fp32) / 64 (bf16);
 * 1: always token by token through the decode kernels. */
int mlh_set_prefill_mode(mlh_ctx* ctx, int mode);

/* One greedy decode step for sequences 0..nseq-1: feeds last_ids[s] at each
 * sequence's current position, appends it, returns argmax of the logits
 * (lowest index on ties) in next_ids[s].  Replaces one iteration of the loop
 * body inference_orchestrator.cu:64-154 (runInference + D2H of vocab*L floats
 * + host qsort + H2D of the ids). */
int mlh_decode_step(mlh_ctx* ctx, const int32_t* last_ids, int nseq, int32_t* next_ids);

/* `steps` greedy steps without returning to the host in between: the argmax of
 * step i is fed to step i+1 on the device.  out_ids is [steps, nseq].
 * Replaces the whole while loop of inference_orchestrator.cu:64-160. */
int mlh_decode_loop(mlh_ctx* ctx, const int32_t* first_ids, int nseq, int steps, int32_t* out_ids);

/* Greedy pick (argmax of the logits, lowest index on ties) made on the device
 * for the last position of seq that went through the LM head: the element the
 * reference takes after its host qsort (inference_orchestrator.cu:84,112). */
int mlh_greedy_token(mlh_ctx* ctx, int seq, int32_t* id);

/* Logits [vocabSize] of the last position processed for seq
 * (vocabScores_DEVICE, network_globals.h:170; the reference copies
 * probabilities for all L positions, inference_orchestrator.cu:68-69). */
int mlh_read_logits(mlh_ctx* ctx, int seq, float* out);

/* Softmax of those logits (vocabScores_postSoftmax_DEVICE, inference.cu:745-749). */
int mlh_read_probs(mlh_ctx* ctx, int seq, float* out);

/* How the kernel-sequence decode step is issued: 0 = plain kernel launches (default); k >= 1 = replays
 * of a captured hipGraph that covers k consecutive decode steps (at most 64). */
int mlh_set_graph(mlh_ctx* ctx, int stepsPerGraph);

/* Batch-1 decode (nseq = 1): mode 1 runs, when the shape allows it, as ONE launch of a
 * persistent kernel (one workgroup per compute unit) that decodes all requested steps: the ~60
 * dependent phases of a token are separated by grid barriers instead of kernel launches.
 * Mode 3 treats each of the eight XCDs as a tensor-parallel rank (heads and FFN units are split over the
 * XCDs, exchanges inside an XCD go through its L2, only two per layer cross XCDs); it covers models with
 * head size 64 (attention heads; gated-delta-net heads with 64 x 64 states, as many as attention heads;
 * per-layer embeddings of a width that is a multiple of 8) and attention-only models with head size 128 (the
 * reference's compiled-in shape, network_meta.h:3-20: 6 heads x 128) on a 256-unit device
 * (mlh_xcd_decode_supported), and falls back to mode 1 otherwise.  Mode 3 is the default.
 * Both need every compute unit for themselves and all their waits are bounded: when a launch gives up (units held
 * by other work), the sequence is as it was before the launch (position, token and tags are written at a kernel's
 * normal end only; the XCD-rank kernel keeps gated-delta-net states in LDS until then, the barrier kernel's are put
 * back from a copy taken before its launch), and the call redoes its steps as the kernel sequence and
 * leaves the context at mode 0 (mlh_get_persistent, mlh_persistent_fallbacks).
 * Mode 0, unsupported shapes and nseq > 1: a sequence of kernels issued as mlh_set_graph says. */
int mlh_set_persistent(mlh_ctx* ctx, int mode);

/* The mode in effect (it differs from what mlh_set_persistent was given after a fallback), and how many decode
 * calls so far were started as a single launch, gave up a wait and were redone as the kernel sequence.  After such
 * a call the context stays at mode 0; mlh_last_error keeps the reason. */
int mlh_get_persistent(mlh_ctx* ctx);
int mlh_persistent_fallbacks(mlh_ctx* ctx);

/* Test hooks (no counterpart in the reference).  mlh_debug_inject_abort: the next `launches` single-launch decode
 * launches find their bounded wait already given up (XCD-rank kernel: arrival counters that start full; barrier
 * kernel: an abort flag that starts raised), so every workgroup leaves at once and the fallback path runs without
 * any wait having to expire.  mlh_debug_set_xcd_tag: sets the XCD-rank kernel's running tag count (device word and
 * host mirror), to exercise the reset that precedes a wrap of the 32-bit tags. */
int mlh_debug_inject_abort(mlh_ctx* ctx, int launches);
/* mlh_debug_inject_abort_at_step: the next single-launch decode launch gives up by itself when workgroup 0 reaches
 * decode step `step` (> 0; counted from 0 inside the launch) -- after the earlier steps have run and written what
 * they write -- so the test can see that the redo starts from the state before the launch.  0 switches it off. */
int mlh_debug_inject_abort_at_step(mlh_ctx* ctx, int step);
int mlh_debug_set_xcd_tag(mlh_ctx* ctx, unsigned tagsUsed);

/* Next-token rule of the decode entry points.  temperature 0 (the default): greedy, the argmax fused into the
 * LM-head reduction, lowest index on ties (the reference's only mode: it keeps the top entry of a qsort of the
 * probabilities, inference_orchestrator.cu:120-165).  temperature > 0: the token is drawn on the device from
 * softmax(logits / temperature) -- the smallest index whose cumulative probability exceeds u, with u a 53-bit
 * uniform from a counter-based generator (SplitMix64) keyed by (seed, sequence id, position of the drawn token), so
 * a sequence draws the same tokens alone, in a batch or from a graph.  Sampling has no counterpart in the
 * reference.  While it is on, batch-1 decode runs as the kernel sequence (the single-launch modes fuse the argmax
 * only).  Returns 0, or -1 for a temperature outside [0, 1e4]. */
int mlh_set_sampling(mlh_ctx* ctx, float temperature, unsigned long long seed);

/* 1 when mode 3 of mlh_set_persistent applies to this context's model and device, else 0
 * (no counterpart in the reference: its decode loop is one kernel sequence, inference_orchestrator.cu:120-165). */
int mlh_xcd_decode_supported(mlh_ctx* ctx);

int mlh_synchronize(mlh_ctx* ctx);

/* Measurement support.  Times `iters` back-to-back launches of one kernel of
 * the decode step with HIP events on the context's stream and returns the
 * average duration in microseconds plus the algorithmic bytes one launch moves. */
enum {
    MLH_K_QKV = 0,
    MLH_K_ATTN = 1,
    MLH_K_OPROJ = 2,
    MLH_K_FFN_GATEUP = 3,
    MLH_K_FFN_DOWN = 4,
    MLH_K_LMHEAD = 5,
    MLH_K_GDN = 6,
    MLH_K_COPY = 7, /* plain copy of nbytes (calibration of the traffic counters) */
    MLH_K_EMBED = 8,
    MLH_K_FINISH = 9,
    MLH_K_COUNT = 10
};
int mlh_time_kernel(mlh_ctx* ctx, int kernel, int layer, int nseq, int iters, double* avg_us,
                    double* algo_bytes);
const char* mlh_kernel_name(int kernel);

/* In-sequence kernel times: runs `steps` decode steps as plain launches with a HIP event after
 * every kernel on the context's stream and returns, per kernel id, the mean time from the previous
 * event to its own (its run time plus the launch gap before it) in us_per_launch[MLH_K_COUNT] and
 * the launches per step in launches_per_step[MLH_K_COUNT].  The sequences advance by `steps`. */
int mlh_profile_decode(mlh_ctx* ctx, const int32_t* first_ids, int nseq, int steps, double* us_per_launch,
                       int32_t* launches_per_step);

/* Latency of one dependent exchange between workgroups on this device, the quantity that bounds batch-1 decode
 * (a token is a chain of about 60 all-to-all exchanges): microseconds per round, over `iters` dependent rounds in
 * one launch of one workgroup per compute unit, of us[0] an all-to-all of `dim` tagged words among the workgroups
 * of one XCD through its L2, us[1] the same among all workgroups through the memory side, us[2] a two-level grid
 * barrier of relaxed atomics.  A figure of -1 means that probe's bounded wait expired.  Measurement support; no
 * counterpart in the reference. */
int mlh_probe_hops(mlh_ctx* ctx, int iters, double* us);

/* Two yardsticks under the prefill GEMM's ceiling (measurement support; no counterpart in the reference, nothing on
 * the product path calls them).  mlh_probe_mfma: TFLOP/s of a register-only half-precision MFMA loop on every SIMD
 * of the device (no LDS, no memory): form 0 = v_mfma_f32_32x32x16_f16, 1 = v_mfma_f32_16x16x32_f16; data 0 =
 * all-zero operands, 1 = pseudo-random operands of unit variance; `iters` loop iterations of 16 (form 0) or 32
 * (form 1) MFMAs per wave, eight waves per compute unit.  The part sets its clock by the power the data draws, so
 * the four figures say how much of the nominal peak each instruction form keeps on real operands.
 * mlh_probe_lds_loads: TB/s of the GEMM's direct global -> LDS load pattern alone (every workgroup streams `slices`
 * 64 KB K slices into LDS, operands resident in its XCD's L2, nothing multiplied). */
int mlh_probe_mfma(mlh_ctx* ctx, int form, int data, int iters, double* tflops);
int mlh_probe_lds_loads(mlh_ctx* ctx, int slices, double* tb_per_s);

/* Times `steps` decode steps (graph replays, argmax fed back on the device)
 * with HIP events on the context's stream: total milliseconds. */
int mlh_time_decode(mlh_ctx* ctx, const int32_t* first_ids, int nseq, int steps, double* total_ms);

/* Stand-alone run of the MFMA GEMM used by prefill and batched decode (no context needed):
 * C[M,N] = A[M,K] . B[N,K]^T (+ R[M,N]), host fp32 arrays in and out; with MLH_DTYPE_BF16 (or 2 = IEEE half) both
 * operands are rounded to that type first.  K*4 (fp32) or K*2 (bf16, half) must be a multiple of 128.
 * dtype | 0x100 selects the SwiGLU epilogue of the gate/up projection instead (R must be null, N even): columns 2j and
 * 2j+1 of the product are gate and up of unit j and C is [M, N/2] with C[m, j] = silu(gate) * up, rounded to the
 * operand type as the prefill pass stores it (inference.cu:262-281).
 * iters > 0 additionally times that many launches with HIP events (mean microseconds in avg_us).
 * Replaces nothing in the reference by itself: it exposes the kernel that stands in for the
 * cublasGemmEx calls of inference.cu:401-743 so that it can be checked and measured alone. */
int mlh_selftest_gemm(int dtype, int M, int N, int K, const float* A, const float* B, const float* R, float* C,
                      int iters, double* avg_us);

/* The same product, C[M,N] = A[M,K] . B[N,K]^T (+ R[M,N]), for callers that cannot allocate -- code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose GEMMs are
 * cuBLAS calls on buffers from allocateMemory).  dA, dB, dR (may be null) and dC are DEVICE pointers on the current
 * device: A and B in the operand type (MLH_DTYPE_F32 float, MLH_DTYPE_BF16 bf16, 2 = IEEE half), R and C fp32, all
 * dense row-major; the launch is enqueued on `stream` (a hipStream_t; null = the default stream) and the call returns
 * without synchronising.  The call allocates and frees nothing: the split-K workspace (tile counters and partial
 * tiles) that mlh_selftest_gemm allocates per call lives here in a static device array of 4 KiB + 2 MiB, which every GPU
 * the library runs on holds until the process ends.  Limits: M <= 64, N <= 32768, K <= 65536, K * element size a
 * multiple of 128 bytes; anything else returns -1 with a message in mlh_last_error(NULL).  All calls on one GPU share
 * that array: calls that may overlap on one GPU (different streams or threads) race and must be ordered by the caller.
 * mlh_gemm_device_init(device) looks up the array's address on that device ahead of time (mlh_create does it too);
 * otherwise the first call on a device does. */
int mlh_gemm_device_init(int device);
int mlh_gemm_device(int dtype, int M, int N, int K, const void* dA, const void* dB, const float* dR, float* dC,
                    void* stream);

#ifdef __cplusplus
}
#endif
#endif
