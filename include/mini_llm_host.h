/*
 * mini_llm_host.h -- host side of the MI355X inference token loop (C ABI).
 *
 * Pure CPU code: model.bin reader/writer, vocab.json tokenizer, story loader,
 * seeded weight/prompt generator and the greedy token loop.  It reaches the
 * GPU only through the device layer of mlh.h.  Each entry cites the reference
 * function whose behaviour it keeps (file:line in daniel-chermetz/mini-llm-cuda).
 * The reference-named C++ functions (loadModel, loadVocab, runInferenceLoop ...)
 * are declared in mini_llm_reference_api.h and are thin wrappers over these.
 *
 * Return conventions follow the reference: loaders return 1 on success and 0
 * on failure (load_model.cu:196-280,474-480); run functions return 0 on
 * success (inference_orchestrator.cu:35-37,188); diagnostics go to stdout.
 */
#ifndef MINI_LLM_HOST_H
#define MINI_LLM_HOST_H

#include <stdint.h>

#include "mlh.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- hyper-parameters --------------------------------------------------- */

/* The compiled-in values of network_meta.h:3-20 (dim 768, 6 heads x 128, ffnDim 3072,
 * 16 layers, maxL 1280, vocab 20160, both architecture flags on). */
void mll_hparams_reference_defaults(mlh_hparams* hp);

/* The five benchmark configurations (1..5).  Returns 1, or 0 for an unknown number. */
int mll_hparams_config(int config, mlh_hparams* hp);

/* Layer kinds for "n GDN : 1 attention" counted in application order (the first
 * applied block is file index transformers-1, inference.cu:384-385): every
 * (gdnPerAttn+1)-th applied block is attention.  gdnPerAttn = 0: all attention. */
void mll_set_layer_pattern(mlh_hparams* hp, int gdnPerAttn);

/* getPreComputedRopeTheta (inference.cu:364-374), with headDim/base as arguments. */
void mll_rope_table(float* tab, int maxL, int headDim, float base);

/* ---- model.bin ---------------------------------------------------------- */

typedef struct mll_model mll_model;

/* Zero-filled model of the given shape (the host half of allocateMemory,
 * memory_allocation.cu:354-499, without its rand() placeholders). */
mll_model* mll_model_new(const mlh_hparams* hp);
void mll_model_free(mll_model* m);
const mlh_hparams* mll_model_hparams(const mll_model* m);

/* Borrowed pointer to a tensor's fp32 data, row-major [rows, cols] as in the
 * file; NULL if the tensor is not part of this model.  layer = file block index. */
float* mll_model_tensor(mll_model* m, int layer, int tensor_id, int* rows, int* cols);

/* Seeded N(0, std) matrices and embedding tables, RMS gains 1, GDN gate biases
 * N(0, 1).  Counter-based generator: element i of a tensor depends only on
 * (seed, layer, tensor id, i).  Replaces initializeRandomWeights
 * (random_weights.cu:34-112), whose cuRAND stream is not reproducible off CUDA. */
void mll_model_init_normal(mll_model* m, uint64_t seed, float std);
/* Uniform [-range, range) instead of normal: the distribution of random_weights.cu:15-25. */
void mll_model_init_uniform(mll_model* m, uint64_t seed, float range);

/* n token ids uniform in [0, vocab) from the same generator (stream selects an
 * independent sequence, e.g. the prompt of sequence `stream`). */
void mll_random_tokens(uint64_t seed, int stream, int vocab, int n, int32_t* out);

/* Reads a checkpoint in the reader convention of load_model.cu:286-481: u64 LE
 * header length, JSON header, data at the next multiple of 8, tensors in the
 * fixed code order, 2-D tensors row-major [out, in], float32 or float64.
 * hint may be NULL when the header carries a "networkMeta" object (written by
 * mll_model_save); otherwise it supplies what shapes cannot (attnHeads, maxL ...).
 * Returns NULL on failure with the reason in err. */
mll_model* mll_model_load(const char* path, const mlh_hparams* hint, char* err, int errLen);

/* Writes that same reader convention (NOT the transposed layout save_model.cu:83-124
 * produces).  float64 != 0 stores doubles.  Returns 1 on success. */
int mll_model_save(const mll_model* m, const char* path, int float64);

/* Uploads every tensor and the RoPE table to a device context and finalizes it.  1 = ok. */
int mll_model_upload(const mll_model* m, mlh_ctx* ctx);

/* ---- vocab.json --------------------------------------------------------- */

typedef struct mll_vocab mll_vocab;

/* loadVocab (load_model.cu:196-280): flat JSON array of strings, index = id.
 * expectSize <= 0: take the array size; otherwise ids >= expectSize are dropped
 * and a size mismatch only warns, as the reference does. */
mll_vocab* mll_vocab_load(const char* path, int expectSize);
void mll_vocab_free(mll_vocab* v);
int mll_vocab_size(const mll_vocab* v);
/* vocabGetToken (load_model.cu:188-193): borrowed pointer or NULL. */
const char* mll_vocab_token(const mll_vocab* v, int index);
/* vocabLookup (load_model.cu:174-185): id or -1. */
int mll_vocab_lookup(const mll_vocab* v, const char* token);
/* hashToken (load_model.cu:153-160): DJB2 through plain char, modulo 20011. */
unsigned int mll_hash_token(const char* str);

/* ---- prompt loader ------------------------------------------------------ */

/* loadStoryContext (main.cu:45-175): JSON array of arrays of token strings;
 * context length max(1, total*percentage/100) capped at maxL+1; ids into out
 * (capacity maxL+1).  Returns the count, 0 on any failure. */
int mll_load_story_context(const char* storiesPath, int storyIndex, int percentage, const mll_vocab* v,
                           int maxL, int32_t* out);

/* loadStoriesFromFile (training_orchestrator.cu:103-273): ALL stories of a tokenised-stories file.
 * Story i that loads occupies tokens[i*(maxL+1) .. (i+1)*(maxL+1)): its first min(count, maxL+1) ids, then
 * MLL_PADDING_TOKEN_INDEX; rightEnd[i] = ids loaded - 2 (the last position with a known next token, so the
 * forward runs over L = rightEnd[i]+1 positions).  At most maxStories stories of the file are looked at
 * (the reference's MAX_TRAINING_STORIES); stories that are not arrays, are empty, have fewer than two
 * tokens, or hold a non-string or out-of-vocabulary token are skipped with a warning.  Returns the number
 * of stories loaded, 0 for an empty file, -1 on error (missing file, not JSON, not an array). */
#define MLL_PADDING_TOKEN_INDEX 89   /* training_orchestrator.h:11 */
#define MLL_MAX_TRAINING_STORIES 2000 /* training_orchestrator.h:6 */
int mll_load_stories(const char* filePath, const mll_vocab* v, int maxL, int maxStories, int32_t* tokens,
                     int32_t* rightEnd);

/* Feeds `count` loaded stories (slab and rightEnd as mll_load_stories fills them, first story `first`) to
 * the device in ONE batched prefill: story first+i is appended to sequence i (which the call empties first)
 * over its L = rightEnd+1 positions.  The context needs maxSeqs >= count.  Returns 0, or -1 on error. */
int mll_prefill_stories(mlh_ctx* ctx, const int32_t* tokens, const int32_t* rightEnd, int maxL, int first,
                        int count);

/* The forward half of processSequence (training_orchestrator.cu:289-359) for one loaded story: a
 * teacher-forced forward over L = rightEnd+1 positions on sequence 0, then for every position whose next
 * token is not the padding token: loss += -logf(max(p(next), 1e-4)).  story points at the story's maxL+1
 * ids.  Returns 0 and fills totalLoss / numPredictions (either may be null); non-zero on error. */
int mll_story_loss(mlh_ctx* ctx, const int32_t* story, int rightEnd, float* totalLoss, int* numPredictions);

/* ---- token loop --------------------------------------------------------- */

typedef struct {
    int tokenIdx;
    float prob;
} mll_token_prob; /* TokenProb, inference_orchestrator.h:4-7 */

/* Greedy generation on sequence 0 of ctx: prefill `n` prompt ids, then decode
 * until maxNew tokens were produced or the sequence reaches maxL (the reference
 * stops only at maxL, inference_orchestrator.cu:64).  out receives the new ids;
 * returns their count, or -1 on error.  elapsedMs (optional) covers the decode loop. */
int mll_generate(mlh_ctx* ctx, const int32_t* prompt, int n, int maxNew, int32_t* out, double* elapsedMs);

/* Top-k of the last position's probabilities, sorted descending as
 * compareTokenProb (inference_orchestrator.cu:20-23) orders them; ties by lower id. */
int mll_top_k(mlh_ctx* ctx, int seq, int k, mll_token_prob* out);

#ifdef __cplusplus
}
#endif
#endif
