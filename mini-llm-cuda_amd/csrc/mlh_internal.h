// Internal declarations of the gfx950 device layer (not part of the C ABI).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>
#include <vector>

#include "mlh.h"

#define MLH_KV_PAGE 64      // positions per KV page; equals the attention key tile
#define MLH_ATTN_WG_KEYS 256 // keys one attention workgroup covers (4 waves x one 64-key tile)
#define MLH_WAVE 64

typedef uint16_t bf16_t;
// IEEE half, as the MFMA path stores weights and activations of bf16 models (see MLH_GEMM_F16)
struct f16_t { uint16_t bits; };
#define MLH_GEMM_F16 2 // GEMM operand type code beside MLH_DTYPE_F32 / MLH_DTYPE_BF16
#define MLH_SELFTEST_SWIGLU 0x100 // mlh_selftest_gemm: flag beside the operand type, selects the SwiGLU epilogue

// Device-side description of one transformer block.
struct LayerDev {
    const void* Wa;       // fused first-phase matrix [rowsA, dim]: q|k|v|[g]|[pleGate]|[gdnA|gdnB]
    const void* Wo;       // [dim, ad]
    const void* W13;      // [2*ffnDim, dim], row 2i = gate row i, row 2i+1 = up row i
    const void* W2;       // [dim, ffnDim]
    const void* pleUp;    // [dim, pleDim]
    const void* pleTable; // [vocab, pleDim]
    const float* g1;      // rms1 gain
    const float* g2;      // rms2 gain
    const float* gq;      // per-head q gain [dim] (qkRmsNorm)
    const float* gk;
    const float* gdnBa;   // [gdnHeads]
    const float* gdnBb;
    float* K;             // KV page pools [numPages, MLH_KV_PAGE, dim]
    float* V;
    float* S;             // GDN states [maxSeqs, gdnHeads, dv, dk]
    int kind;
    int rowsA, offK, offV, offG, offPle, offGa, offGb;
    int ad;               // width of the mixing output fed to Wo
    // What the MFMA path multiplies: the matrices themselves for fp32 models; for bf16 models IEEE-half
    // mirrors scaled by a power of two (exact), with the inverse scale applied to the product.
    // WoG is [dim, ad + pleDim]: Wo with pleUp appended along K, so that h1 = [a | e] . WoG^T is one product.
    const void *WaG, *WoG, *W13G, *W2G;
    float sWa, sWo, sW13, sW2;
};

// Arguments shared by all kernels of a decode step.
struct StepArgs {
    // model
    int dim, heads, hd, ffn, vocab, maxL, ple;
    int gdnHeads, gdnDk, gdnDv;
    int qkNorm, gating;
    // batch
    int nseq;             // active slots
    const int* sidx;      // slot -> sequence id
    const int* tok;       // per slot: token fed this step
    int* pos;             // per sequence: current length (position of the fed token)
    const int* pageTable; // [maxSeqs, pagesPerSeq]
    int pagesPerSeq;
    int nsplit;           // attention partials per (slot, head)
    // activations, indexed by slot
    float* x;             // [slots, dim] residual stream
    float* qkv;           // [slots, maxRowsA]
    int qkvStride;
    float* part;          // [slots, nsplit, heads, hd + 2] attention partials (m, l, acc)
    float* mix;           // [slots, maxAd] GDN read-out
    void* mixRows;        // batched step: if set, the GDN read-out and the PLE columns go straight into the rows of the
    int mixRowsLd;        //   output-projection GEMM (leading dimension in elements, fp32 or IEEE half) instead of `mix`
    int mixRowsHalf;
    int wbytes;           // bytes per weight element (PLE table rows)
    float temperature;    // > 0: the next token is drawn from softmax(logits / temperature) instead of the argmax
    unsigned long long sampleSeed;
    float* h1;            // [slots, dim]
    float* u;             // [slots, ffn]
    float* logits;        // [maxSeqs, vocab] indexed by sequence id
    float* amaxVal;       // [slots, amaxParts]
    int* amaxIdx;
    int amaxParts;
    const float* rope;    // [maxL, hd]
    const void* E;        // [vocab, dim]
    const float* gF;
    int* nextTok;         // [maxSeqs] greedy pick per sequence id
    int* outIds;          // [maxSteps, slots]
    int* stepCounter;
    int outCapacity;
};

struct mlh_ctx {
    mlh_hparams hp;
    int device = 0;
    hipStream_t stream = nullptr;
    std::string err;
    bool finalized = false;
    int wbytes = 4; // bytes per matrix element

    std::vector<LayerDev> layers;
    std::vector<std::vector<char>> have; // [layer][tensor] uploaded flags
    bool haveE = false, haveGF = false, haveRope = false;
    std::vector<void*> allocs;

    void* E = nullptr;
    float* gF = nullptr;
    float* rope = nullptr;

    void* mixRows = nullptr; // see StepArgs::mixRows; set by the batched step around its GDN launches
    int mixRowsLd = 0, mixRowsHalf = 0;
    int pagesPerSeq = 0;
    int nsplit = 1;
    int maxRowsA = 0, maxAd = 0;
    int amaxParts = 0;
    int outCapacity = 0;

    int* d_sidx = nullptr;
    int* d_tok = nullptr;
    int* d_pos = nullptr;
    int* d_pageTable = nullptr;
    int* d_outIds = nullptr;
    int* d_next = nullptr;
    int* d_stepCounter = nullptr;
    int* d_prompt = nullptr;
    int promptCapacity = 0;
    float *x = nullptr, *qkv = nullptr, *part = nullptr, *mix = nullptr, *h1 = nullptr, *u = nullptr;
    float *logits = nullptr, *amaxVal = nullptr, *probs = nullptr;
    int* amaxIdx = nullptr;
    void* copySrc = nullptr; // calibration buffers for MLH_K_COPY
    void* copyDst = nullptr;
    size_t copyBytes = 0;

    // persistent batch-1 decode kernel
    int numCUs = 0;
    bool coopLaunch = false;
    float temperature = 0.f;       // 0: greedy; > 0: temperature sampling (kernel-sequence and batched paths)
    unsigned long long sampleSeed = 0;
    int usePersistent = 3;         // 0: kernel sequence; 1: persistent kernel with grid barriers;
                                   // 3: XCD ranks where the model and device allow it, else as 1
    int persistentFallbacks = 0;   // single-launch decode calls that gave up a wait and were redone as the kernel sequence
    int injectAbort = 0;           // test hook: the next n single-launch decode launches give up at their start
    int injectAbortStep = 0;       // test hook: the next single-launch decode launch gives up when it reaches this step (> 0)
    bool persistCooperative = false; // MLH_PERSIST_COOPERATIVE, read once at creation: cooperative launch of the barrier kernel
    float* gdnSnapshot = nullptr;  // barrier kernel: sequence 0's GDN states as they were before the launch
    unsigned long long xcdTagNext = 0; // host mirror of the XCD-rank kernel's tag counter (tags used so far)
    bool xcdPrepared = false;      // function attribute and occupancy of the XCD-rank kernel checked
    bool persistentPrepared = false;
    int xcdWide = 1, xcdNapRound = 0, xcdNap[5] = {44, 0, 0, 0, 0}; // tuning knobs, read from the environment once at creation
    unsigned long long* xcdBuf = nullptr; // (value, tag) exchange words of mode 3
    size_t xcdWords = 0;
    LayerDev* d_layers = nullptr;  // device copy of `layers`
    unsigned* d_sync = nullptr;    // barrier words + abort flag
    float* pamaxVal = nullptr;     // [numCUs]
    int* pamaxIdx = nullptr;
    float* kvPart = nullptr;       // [heads, pagesPerSeq, headDim + 2]
    unsigned long long* d_timing = nullptr; // phase timestamps (set MLH_PERSIST_TIMING=1), 16 per layer

    std::vector<hipEvent_t>* profEvents = nullptr; // set while mlh_profile_decode runs
    std::vector<int>* profIds = nullptr;

    // prefill work buffers, sized on first use for the largest row count seen
    int pfRows = 0, pfBlkCap = 0;
    int prefillMode = 0; // 0: GEMM path when the shape allows and the call is long enough; 1: token by token
    std::vector<void*> pfAllocs;
    float *pfX = nullptr, *pfQKV = nullptr, *pfH1 = nullptr;
    void *pfXn = nullptr, *pfA = nullptr, *pfU = nullptr;
    uint16_t *pfKh = nullptr, *pfVh = nullptr; // half copies of a call's K and V rows for the MFMA attention of a fresh prefill
    int* pfMeta = nullptr;
    int pfChunkCap = 0;
    void* pfGdnWs = nullptr;   // chunk operands of the chunk-parallel GDN prefill
    float* pfGdnG = nullptr;
    size_t pfGdnChunks = 0;
    const void* EG = nullptr;  // LM-head matrix as the MFMA path reads it (see LayerDev::WaG)
    float sE = 1.0f;
    int gemmDtype = MLH_DTYPE_F32; // operand type of the MFMA path: MLH_DTYPE_F32 or MLH_GEMM_F16
    std::vector<void*> mirrorAllocs;
    long f16Inexact = 0;       // bf16 weights that had no exact scaled-half representation (reported at finalize)
    void* gemmWs = nullptr;    // split-K workspace of the skinny GEMM
    float* pfLogits = nullptr; // [64, vocab] logits of a batched decode step in slot order

    std::vector<int> h_len; // host mirror of d_pos
    int identityNseq = 0;   // d_sidx currently holds 0..identityNseq-1 (0 = unknown)

    int graphSteps = 0;                 // 0: eager launches; k >= 1: one graph replay covers k decode steps
    hipGraphExec_t graphExec[2] = {};   // [0]: one step, [1]: graphSteps steps
    int graphNseqOf[2] = {0, 0};
    int graphStepsOf[2] = {0, 0};
};

// kernels_decode.hip
int mlh_launch_step(mlh_ctx* c, int nseq, const int* tokPtr, bool lmHead);
int mlh_launch_one(mlh_ctx* c, int kernel, int layer, int nseq);
double mlh_kernel_bytes(mlh_ctx* c, int kernel, int layer, int nseq);
void mlh_fill_args(mlh_ctx* c, StepArgs& a, int nseq, const int* tokPtr);
int mlh_launch_copy(mlh_ctx* c);
int mlh_dev_alloc_bytes(mlh_ctx* c, void** p, size_t bytes); // mlh_api.hip: an allocation owned by the context
int mlh_launch_probs(mlh_ctx* c, int seq);
int mlh_init_kernels(mlh_ctx* c);

// kernels_gemm.hip
hipError_t mlh_gemm_tn(hipStream_t stream, int dtype, const void* A, int lda, const void* B, int ldb, float* C, int ldc,
                       const float* R, int ldr, int M, int N, int K);
// epi 0: as above.  epi 1 (SwiGLU): columns 2j / 2j+1 of the product are gate / up of unit j and
// C is [M, N/2] in the operand type: C[m, j] = silu(gate) * up.
// ws: zero-initialised workspace of mlh_gemm_workspace_bytes() or null; with it, M <= 64 products of matrices
// with few rows are split along K over workgroups (deterministically reduced).
// alpha scales the product before the epilogue (the power of two an fp16 weight mirror was scaled by, inverted).
// normGain (M <= 64 for fp32 operands, M <= 32 for half operands, see mlh_gemm_norm_fusable): A holds the raw fp32
// rows -- also when the weights are half -- and the product is taken of gain * A / rms(A) (the RMSNorm of the rows,
// eps 1e-8 inside the root), without a pass that writes the normalised rows.
hipError_t mlh_gemm_tn_epi(hipStream_t stream, int dtype, int epi, const void* A, int lda, const void* B, int ldb, void* C, int ldc,
                           const float* R, int ldr, int M, int N, int K, void* ws, float alpha = 1.0f, const float* normGain = nullptr);
bool mlh_gemm_norm_fusable(int dtype, int M, int N, int K);
size_t mlh_gemm_workspace_bytes(void);
extern "C" int mlh_gemm_device_init(int device);

// mlh_api.hip: message returned by mlh_last_error(NULL) on this thread (context-free entry points)
void mlh_set_thread_error(const std::string& msg);

// kernels_prefill.hip
bool mlh_prefill_gemm_supported(const mlh_ctx* c);
int mlh_init_prefill_kernels(mlh_ctx* c);
int mlh_build_gemm_operands(mlh_ctx* c); // at finalize: fp16 mirrors for bf16 models
bool mlh_batch_step_applicable(const mlh_ctx* c, int nseq);
int mlh_prepare_batch_step(mlh_ctx* c, int nseq);
int mlh_launch_batch_step(mlh_ctx* c, int nseq, const int* tokPtr);
int mlh_run_prefill_gemm(mlh_ctx* c, int nseg, const int32_t* seqs, const int32_t* ids, const int32_t* lens, float* allLogits);
int mlh_launch_softmax_rows(mlh_ctx* c, const float* logits, float* probs, const int* target, float* nll, int rows);

// kernels_persistent.hip
bool mlh_persistent_supported(const mlh_ctx* c);
int mlh_launch_persistent(mlh_ctx* c, int steps);
int mlh_persistent_restore_states(mlh_ctx* c);

// measure_timing.hip: decodes and prints the phase clock stamps of the single-launch decode kernels
// (collected only when MLH_PERSIST_TIMING is set at context creation)
void mlh_dump_persistent_timing(mlh_ctx* c);

// kernels_xcd.hip
size_t mlh_xcd_words(const mlh_ctx* c);
bool mlh_xcd_supported(const mlh_ctx* c);
int mlh_xcd_reset(mlh_ctx* c);
int mlh_launch_xcd(mlh_ctx* c, int steps);

#define MLH_CHECK(ctx, expr)                                                               \
    do {                                                                                   \
        hipError_t e_ = (expr);                                                            \
        if (e_ != hipSuccess) {                                                            \
            (ctx)->err = std::string(#expr) + ": " + hipGetErrorString(e_);                \
            return -2;                                                                     \
        }                                                                                  \
    } while (0)
