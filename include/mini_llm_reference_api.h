/*
 * mini_llm_reference_api.h -- the reference's own inference-path surface, kept
 * name for name (C++ linkage, process-wide state, same return conventions), so
 * that code written against daniel-chermetz/mini-llm-cuda links against this
 * library unchanged.  Everything here is a thin wrapper over mini_llm_host.h
 * and mlh.h.
 *
 * The reference fixes its shape at compile time (network_meta.h:3-20).  Here
 * the same names are runtime fields of mlh_hparams: call mllSetNetworkMeta()
 * before allocateMemory() to run another shape; without it the reference's
 * compiled-in values apply.
 */
#ifndef MINI_LLM_REFERENCE_API_H
#define MINI_LLM_REFERENCE_API_H

#include "mini_llm_host.h"

/* network_globals.h:147: host copy of the token ids, maxL+1 entries after allocateMemory(). */
extern int* seqTokenIndices;

typedef mll_token_prob TokenProb; /* inference_orchestrator.h:4-7 */

/* memory_allocation.h:5.  Allocates the device context for the current network meta
 * (inference buffers only; the flag is accepted and ignored). */
void allocateMemory(bool allocateTraining);

/* load_model.h:3-6 */
int loadVocab(const char* vocabPath);
char* vocabGetToken(int index);
int vocabLookup(const char* token);
int loadModel(const char* modelName); /* opens ./model/<modelName>.bin */

/* random_weights.h:4 (uniform in [-range, range), gains 1, seed 42). */
void initializeRandomWeights(float range);

/* inference.h:3-4.  runInference(L) consumes seqTokenIndices[0..L) and leaves the
 * last position's logits/probabilities readable through mllDeviceContext(). */
int runInference(int L);
/* The same forward over all L positions from scratch, with the contents of
 * vocabScores_postSoftmax_DEVICE (network_globals.h:172-174: [vocabSize x L], position i at
 * i * vocabSize) copied to hostProbs and the sequence loss of processSequence
 * (training_orchestrator.cu:289-359) to meanLoss; either may be null.  0 = success. */
int runInferenceAllPositions(int L, float* hostProbs, float* meanLoss);
void getPreComputedRopeTheta(float* preComputedRopeTheta, int maxL_);

/* main.cu:45 (declared extern in inference_orchestrator.cu:26) */
int loadStoryContext(const char* storiesPath, int storyIndex, int percentage);

/* inference_orchestrator.h:17-18 */
int runInferenceLoop(const char* storiesPath, int storyIndex, int contextPercent, bool skipUserInput,
                     bool verboseOutput);

/* ---- additions (no counterpart in the reference) ---- */
void mllSetNetworkMeta(const mlh_hparams* hp);
const mlh_hparams* mllGetNetworkMeta();
int loadModelFile(const char* filepath); /* loadModel with an explicit path */
mlh_ctx* mllDeviceContext();
void mllShutdown(); /* frees what the reference leaves to process exit */

#endif
