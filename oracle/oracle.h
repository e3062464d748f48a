/*
 * CPU oracle for the mini-llm inference token loop.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing on the product path (the HIP library, the
 * C++ host library, their Python bindings) may call, link or import this code.
 * It exists so that tests, the smoke check and the benchmark's CPU-baseline leg
 * have an independent statement of the arithmetic to compare the GPU against.
 *
 * What it restates (reference file:line):
 *   - embedding gather                      inference.cu:9-22
 *   - RMSNorm (eps inside the sqrt)         inference.cu:24-50, 83-95
 *   - per-head Q/K RMSNorm                  inference.cu:52-81, 97-111
 *   - RoPE table and rotation               inference.cu:113-134, 364-374
 *   - masked, scaled KtQ, softmax, V.P      inference.cu:136-239, 511-573
 *   - sigmoid query gating                  inference.cu:241-250
 *   - residual adds, SiLU, Hadamard         inference.cu:252-291
 *   - final norm, tied LM head, softmax     inference.cu:293-362, 705-749
 *   - layer order (file index 0 = top)      inference.cu:384-385
 *   - greedy pick                           inference_orchestrator.cu:77-84,112
 *
 * Parts with no counterpart in the reference (KV cache, gated-delta-net layer,
 * per-layer embeddings) follow the definitions written at each function below;
 * they are pinned by closed forms and invariants in tests/, not by reference
 * vectors, because the reference holds none.
 *
 * Parity status: the reference ships no numeric golden outputs, and its GEMMs
 * go through cuBLAS in TF32 mode (main.cu:179), so agreement with the CUDA
 * binary's numbers is "parity unpinned".  Every function here is pinned
 * against closed forms / brute force / an independent NumPy restatement
 * (tests/test_oracle_pins.py): the per-layer-embedding branch by
 * x + Wpu (silu(Wpg xn) * P[tok]) on a one-block model plus a table-row swap,
 * the gated-delta-net gates and update by their matrix form on two tokens,
 * the blocked product of the full-sequence forward by bit-equality with the
 * one-vector product.
 *
 * Every function exists twice: suffix _f32 computes in float (the reference's
 * type), suffix _f64 in double (the arbiter for tolerance decisions).
 */
#ifndef ORACLE_H
#define ORACLE_H

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_MAX_LAYERS 64
#define ORC_KIND_ATTENTION 0
#define ORC_KIND_GDN 1

/* Runtime form of network_meta.h:3-20; names follow the macros. */
typedef struct {
    int dim;
    int attnHeads;
    int headDim;
    int ffnDim;
    int transformers;
    int maxL;
    int vocabSize;
    float ropeDenomBase;
    int qkRmsNorm;    /* CONFIG_QK_RMS_NORM  (attention layers only) */
    int queryGating;  /* CONFIG_QUERY_GATING (attention layers only) */
    int gdnHeads, gdnDk, gdnDv;
    int pleDim;       /* 0 = no per-layer embeddings */
    int layerKinds[ORC_MAX_LAYERS]; /* by FILE index (0 = top of the stack) */
} orc_hparams;

/* All matrices row-major [out, in], i.e. exactly the byte order of model.bin
 * (load_model.cu:87-100 transposes this into cuBLAS column-major; the oracle
 * indexes W[o*in + i] directly, which is the same mathematical matrix). */
typedef struct {
    const float* rms1;   /* [dim] */
    const float* Wq;     /* attention: [dim, dim]; GDN: [gdnHeads*gdnDk, dim] */
    const float* Wk;
    const float* Wv;     /* attention: [dim, dim]; GDN: [gdnHeads*gdnDv, dim] */
    const float* Wo;     /* attention: [dim, dim]; GDN: [dim, gdnHeads*gdnDv] */
    const float* rms2;   /* [dim] */
    const float* W1A;    /* gate, SiLU branch [ffnDim, dim] (ffn_right_1) */
    const float* W1B;    /* up [ffnDim, dim] (ffn_right_2) */
    const float* W2;     /* down [dim, ffnDim] (ffn_left) */
    const float* qRms;   /* [dim] or NULL */
    const float* kRms;   /* [dim] or NULL */
    const float* Wg;     /* [dim, dim] or NULL */
    const float* gdnWa;  /* [gdnHeads, dim] */
    const float* gdnBa;  /* [gdnHeads] */
    const float* gdnWb;  /* [gdnHeads, dim] */
    const float* gdnBb;  /* [gdnHeads] */
    const float* pleTable; /* [vocabSize, pleDim] */
    const float* pleGate;  /* [pleDim, dim] */
    const float* pleUp;    /* [dim, pleDim] */
} orc_layer;

typedef struct {
    const float* E;       /* [vocabSize, dim], token-major */
    const float* gammaF;  /* [dim] */
    orc_layer layers[ORC_MAX_LAYERS];
} orc_weights;

/* RoPE table exactly as inference.cu:364-374 (float powf/cosf/sinf). */
void orc_rope_table(float* tab, int maxL, int headDim, float base);

/* Round-to-nearest-even fp32 -> bf16 -> fp32, in place (bf16-weight path). */
void orc_round_bf16(float* w, long n);

#define ORC_DECL(SFX, REAL)                                                            \
    /* unit ops (exported for per-kernel tests) */                                     \
    void orc_rmsnorm_##SFX(const REAL* x, const float* gamma, int n, REAL* y);         \
    void orc_head_rmsnorm_##SFX(REAL* q, const float* gamma, int heads, int hd);       \
    void orc_rope_##SFX(REAL* q, const float* tab, int pos, int heads, int hd);        \
    void orc_matvec_##SFX(const float* W, const REAL* x, int rows, int cols, REAL* y); \
    void orc_matmat_##SFX(const float* W, const REAL* X, int ldx, int rows, int cols, int L, \
                          REAL* Y, int ldy);                                           \
    void orc_attend_##SFX(const REAL* q, const REAL* K, const REAL* V, int T, int dim, \
                          int heads, int hd, REAL* out);                               \
    void orc_gdn_step_##SFX(REAL* S, const REAL* q, const REAL* k, const REAL* v,      \
                            REAL alpha, REAL beta, int dk, int dv, REAL* o);           \
    /* cached decode */                                                                \
    void* orc_state_new_##SFX(const orc_hparams* hp, const orc_weights* w);            \
    void orc_state_reset_##SFX(void* st);                                              \
    void orc_state_free_##SFX(void* st);                                               \
    int orc_state_pos_##SFX(void* st);                                                 \
    int orc_decode_step_##SFX(void* st, int token, REAL* logits);                      \
    /* reference-style full recompute over L columns */                                \
    int orc_forward_full_##SFX(const orc_hparams* hp, const orc_weights* w,            \
                               const int* tokens, int L, REAL* logits, REAL* probs,    \
                               REAL* finalHidden, int lastOnly);

ORC_DECL(f32, float)
ORC_DECL(f64, double)

#ifdef __cplusplus
}
#endif
#endif
