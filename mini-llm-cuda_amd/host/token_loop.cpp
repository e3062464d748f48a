// Greedy token loop over the device layer, and the reference-named C++ surface
// (mini_llm_reference_api.h) that makes the library a drop-in for the
// reference's inference path.
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <chrono>
#include <vector>

#include "mini_llm_host.h"
#include "mini_llm_reference_api.h"

// ---------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------
extern "C" int mll_generate(mlh_ctx* ctx, const int32_t* prompt, int n, int maxNew, int32_t* out, double* elapsedMs) {
    if (!ctx || !prompt || n <= 0 || !out) return -1;
    auto start = std::chrono::high_resolution_clock::now();
    if (mlh_reset(ctx, 0)) return -1;
    if (mlh_prefill(ctx, 0, prompt, n)) return -1;
    // The reference keeps generating until the sequence holds maxL tokens
    // (inference_orchestrator.cu:64); the last token it appends is never fed back.
    const int room = mlh_max_len(ctx) - n;
    const int G = std::min(maxNew, room);
    int produced = 0;
    if (G >= 1) {
        if (mlh_greedy_token(ctx, 0, &out[0])) return -1;
        produced = 1;
        if (G > 1) {
            if (mlh_decode_loop(ctx, &out[0], 1, G - 1, out + 1)) return -1;
            produced = G;
        }
    }
    auto end = std::chrono::high_resolution_clock::now();
    if (elapsedMs) *elapsedMs = std::chrono::duration<double, std::milli>(end - start).count();
    return produced;
}

extern "C" int mll_top_k(mlh_ctx* ctx, int seq, int k, mll_token_prob* out) {
    if (!ctx || !out || k <= 0) return -1;
    const int V = mlh_vocab_size(ctx);
    if (V <= 0) return -1;
    std::vector<float> probs(V);
    if (mlh_read_probs(ctx, seq, probs.data())) return -1;
    std::vector<int> idx(V);
    for (int i = 0; i < V; i++) idx[i] = i;
    k = std::min(k, V);
    // compareTokenProb (inference_orchestrator.cu:20-23) sorts by descending probability and
    // leaves ties to qsort; ties are resolved here by the lower token id.
    std::partial_sort(idx.begin(), idx.begin() + k, idx.end(), [&](int a, int b) {
        return probs[a] > probs[b] || (probs[a] == probs[b] && a < b);
    });
    for (int i = 0; i < k; i++) { out[i].tokenIdx = idx[i]; out[i].prob = probs[idx[i]]; }
    return k;
}

extern "C" int mll_prefill_stories(mlh_ctx* ctx, const int32_t* tokens, const int32_t* rightEnd, int maxL_,
                                   int first, int count) {
    if (!ctx || !tokens || !rightEnd || first < 0 || count <= 0 || maxL_ != mlh_max_len(ctx)) return -1;
    std::vector<int32_t> seqs(count), lens(count), ids;
    for (int i = 0; i < count; i++) {
        const int L = rightEnd[first + i] + 1;
        if (L < 1 || L > maxL_) return -1;
        seqs[i] = i;
        lens[i] = L;
        const int32_t* story = tokens + (size_t)(first + i) * (maxL_ + 1);
        ids.insert(ids.end(), story, story + L);
        if (mlh_reset(ctx, i)) return -1;
    }
    return mlh_prefill_batch(ctx, count, seqs.data(), ids.data(), lens.data()) ? -1 : 0;
}

extern "C" int mll_story_loss(mlh_ctx* ctx, const int32_t* story, int rightEnd, float* totalLoss, int* numPredictions) {
    if (!ctx || !story || rightEnd < 0 || rightEnd + 1 > mlh_max_len(ctx)) return 1;
    const int L = rightEnd + 1, V = mlh_vocab_size(ctx);
    std::vector<float> probs((size_t)L * V);
    if (mlh_reset(ctx, 0)) return 1;
    if (mlh_forward_full(ctx, 0, story, L, nullptr, probs.data(), nullptr)) return 1;
    float loss = 0.0f;
    int n = 0;
    for (int pos = 0; pos <= rightEnd; pos++) { // training_orchestrator.cu:330-352
        const int next = story[pos + 1];
        if (next == MLL_PADDING_TOKEN_INDEX) continue;
        if (next < 0 || next >= V) return 1;
        float p = probs[(size_t)pos * V + next];
        if (p < 0.0001f) p = 0.0001f;
        loss += -logf(p);
        n++;
    }
    if (totalLoss) *totalLoss = loss;
    if (numPredictions) *numPredictions = n;
    return 0;
}

// ---------------------------------------------------------------------------
// reference-named surface: process-wide state, as network_globals.h:136-174 has it
// ---------------------------------------------------------------------------
int* seqTokenIndices = nullptr;

static mlh_hparams g_hp;
static bool g_hpSet = false;
static mlh_ctx* g_ctx = nullptr;
static mll_model* g_model = nullptr;
static mll_vocab* g_vocab = nullptr;
static std::vector<int> g_cached; // tokens already in the device cache of sequence 0

static const mlh_hparams& current_hp() {
    if (!g_hpSet) { mll_hparams_reference_defaults(&g_hp); mll_set_layer_pattern(&g_hp, 0); g_hpSet = true; }
    return g_hp;
}

void mllSetNetworkMeta(const mlh_hparams* hp) {
    if (hp) { g_hp = *hp; g_hpSet = true; }
}
const mlh_hparams* mllGetNetworkMeta() { return &current_hp(); }
mlh_ctx* mllDeviceContext() { return g_ctx; }

void mllShutdown() {
    if (g_ctx) mlh_destroy(g_ctx);
    g_ctx = nullptr;
    mll_model_free(g_model);
    g_model = nullptr;
    mll_vocab_free(g_vocab);
    g_vocab = nullptr;
    free(seqTokenIndices);
    seqTokenIndices = nullptr;
    g_cached.clear();
}

void allocateMemory(bool /*allocateTraining: the training buffers are not part of this path*/) {
    const mlh_hparams& hp = current_hp();
    if (g_ctx) { mlh_destroy(g_ctx); g_ctx = nullptr; }
    mll_model_free(g_model);
    free(seqTokenIndices);
    seqTokenIndices = (int*)calloc((size_t)hp.maxL + 1, sizeof(int)); // memory_allocation.cu allocates maxL+1 ids
    g_model = mll_model_new(&hp);
    g_cached.clear();
    if (mlh_create(&hp, 0, &g_ctx) != 0) {
        printf("Error: device allocation failed: %s\n", mlh_last_error(nullptr));
        g_ctx = nullptr;
    }
}

void getPreComputedRopeTheta(float* preComputedRopeTheta, int maxL_) {
    const mlh_hparams& hp = current_hp();
    mll_rope_table(preComputedRopeTheta, maxL_, hp.headDim, hp.ropeDenomBase);
}

int loadVocab(const char* vocabPath) {
    mll_vocab_free(g_vocab);
    g_vocab = mll_vocab_load(vocabPath, current_hp().vocabSize);
    return g_vocab ? 1 : 0;
}
char* vocabGetToken(int index) { return const_cast<char*>(mll_vocab_token(g_vocab, index)); }
int vocabLookup(const char* token) { return mll_vocab_lookup(g_vocab, token); }

static int upload_current_model() {
    if (!g_ctx || !g_model) { printf("Error: allocateMemory has not succeeded.\n"); return 0; }
    g_cached.clear();
    if (mlh_reset(g_ctx, -1)) return 0;
    return mll_model_upload(g_model, g_ctx);
}

int loadModel(const char* modelName) {
    char filepath[512];
    snprintf(filepath, sizeof(filepath), "./model/%s.bin", modelName); // load_model.cu:287-288
    return loadModelFile(filepath);
}

int loadModelFile(const char* filepath) {
    char err[256];
    mll_model* m = mll_model_load(filepath, &current_hp(), err, sizeof(err));
    if (!m) { printf("!!! Error loading weights from %s. !!!\n\n", filepath); return 0; }
    mll_model_free(g_model);
    g_model = m;
    return upload_current_model();
}

void initializeRandomWeights(float range) {
    printf("\n=== Initializing Random Weights (range: [-%.4f, +%.4f]) ===\n", range, range);
    if (!g_model) { printf("Error: allocateMemory has not been called.\n"); return; }
    mll_model_init_uniform(g_model, 42, range); // random_weights.cu:37: fixed seed 42
    if (upload_current_model()) printf("=== Random weights initialized ===\n\n");
}

// Processes seqTokenIndices[0..L).  Positions whose tokens are unchanged since
// the previous call stay in the KV cache / GDN state; only the new tail is run.
int runInference(int L) {
    const mlh_hparams& hp = current_hp();
    if (!g_ctx || !seqTokenIndices || L <= 0 || L > hp.maxL) return 1;
    size_t keep = 0;
    while (keep < g_cached.size() && (int)keep < L && g_cached[keep] == seqTokenIndices[keep]) keep++;
    if (keep != g_cached.size() || (int)keep == L) { // diverged, or nothing new: rebuild from the start
        if (mlh_reset(g_ctx, 0)) return 1;
        g_cached.clear();
        keep = 0;
    }
    if (mlh_prefill(g_ctx, 0, seqTokenIndices + keep, L - (int)keep)) {
        printf("Error: %s\n", mlh_last_error(g_ctx));
        return 1;
    }
    g_cached.assign(seqTokenIndices, seqTokenIndices + L);
    return 0;
}

// runInference(L) as the training/verification callers use it (training_orchestrator.cu:289-359): all L
// positions from scratch, probabilities of every position copied out in the layout of
// vocabScores_postSoftmax_DEVICE (position i at hostProbs[i * vocabSize ...]).  hostProbs and meanLoss may be null.
int runInferenceAllPositions(int L, float* hostProbs, float* meanLoss) {
    const mlh_hparams& hp = current_hp();
    if (!g_ctx || !seqTokenIndices || L <= 0 || L > hp.maxL) return 1;
    if (mlh_reset(g_ctx, 0)) return 1;
    g_cached.clear();
    if (mlh_forward_full(g_ctx, 0, seqTokenIndices, L, nullptr, hostProbs, meanLoss)) {
        printf("Error: %s\n", mlh_last_error(g_ctx));
        return 1;
    }
    g_cached.assign(seqTokenIndices, seqTokenIndices + L);
    return 0;
}

int loadStoryContext(const char* storiesPath, int storyIndex, int percentage) {
    const mlh_hparams& hp = current_hp();
    if (!seqTokenIndices) { printf("Error: allocateMemory has not been called.\n"); return 0; }
    return mll_load_story_context(storiesPath, storyIndex, percentage, g_vocab, hp.maxL, seqTokenIndices);
}

static void print_escaped(const char* t) {
    if (!t) return;
    if (strcmp(t, "\n") == 0) printf("[\\n]");
    else if (strcmp(t, "\t") == 0) printf("[\\t]");
    else printf("%s", t);
}

// inference_orchestrator.cu:28-189
int runInferenceLoop(const char* storiesPath, int storyIndex, int contextPercent, bool skipUserInput,
                     bool verboseOutput) {
    const mlh_hparams& hp = current_hp();
    const int maxL_ = hp.maxL;
    int L = loadStoryContext(storiesPath, storyIndex, contextPercent);
    if (L <= 0) { printf("Failed to load story context.\n"); return 1; }
    if (L >= maxL_) {
        printf("Sequence already at maxL=%d tokens (loaded %d). No generation needed.\n", maxL_, L);
        return 0;
    }
    if (!g_ctx) { printf("Error: no device context.\n"); return 1; }
    int tokensGenerated = 0;
    const int maxTokensToGenerate = maxL_ - L;
    printf("\n========================================\n");
    printf("Starting text generation (max %d new tokens)\n", maxTokensToGenerate);
    printf("Press Enter to generate next token, or 'q' + Enter to quit\n");
    printf("========================================\n\n");

    auto start = std::chrono::high_resolution_clock::now();
    if (skipUserInput && !verboseOutput) {
        // Nothing is shown between tokens: the whole loop stays on the device.
        std::vector<int32_t> out(maxTokensToGenerate);
        const int got = mll_generate(g_ctx, seqTokenIndices, L, maxTokensToGenerate, out.data(), nullptr);
        if (got < 0) { printf("Error: %s\n", mlh_last_error(g_ctx)); return 1; }
        for (int i = 0; i < got; i++) seqTokenIndices[L++] = out[i];
        tokensGenerated = got;
        g_cached.assign(seqTokenIndices, seqTokenIndices + L - 1);
    } else {
        while (L < maxL_) {
            if (runInference(L)) return 1;
            int nextTokenIdx = 0;
            if (mlh_greedy_token(g_ctx, 0, &nextTokenIdx)) return 1;
            if (verboseOutput) {
                mll_token_prob top[10];
                const int k = mll_top_k(g_ctx, 0, 10, top);
                printf("\n--- Top 10 Most Probable Next Tokens (position %d) ---\n", L);
                for (int i = 0; i < k; i++) {
                    const char* tokenStr = vocabGetToken(top[i].tokenIdx);
                    if (!tokenStr) continue;
                    if (strcmp(tokenStr, "\n") == 0) printf("%2d. [\\n]         (idx: %5d, prob: %.6f)\n", i + 1, top[i].tokenIdx, top[i].prob);
                    else if (strcmp(tokenStr, "\t") == 0) printf("%2d. [\\t]         (idx: %5d, prob: %.6f)\n", i + 1, top[i].tokenIdx, top[i].prob);
                    else if (strlen(tokenStr) == 0) printf("%2d. [EMPTY]       (idx: %5d, prob: %.6f)\n", i + 1, top[i].tokenIdx, top[i].prob);
                    else printf("%2d. %-12s (idx: %5d, prob: %.6f)\n", i + 1, tokenStr, top[i].tokenIdx, top[i].prob);
                }
                printf("-------------------------------------------------------\n");
                printf("\nMost probable token: ");
                print_escaped(vocabGetToken(nextTokenIdx));
                printf(" (index: %d)\n", nextTokenIdx);
            }
            if (!skipUserInput) {
                printf("\nPress Enter to add this token and continue, or 'q' + Enter to quit: ");
                fflush(stdout);
                char input[10];
                if (fgets(input, sizeof(input), stdin) == NULL) break;
                if (input[0] == 'q' || input[0] == 'Q') { printf("Generation stopped by user.\n"); break; }
            }
            seqTokenIndices[L] = nextTokenIdx;
            L++;
            tokensGenerated++;
            if (verboseOutput) printf("\n[Token added. Total context: %d tokens, generated: %d]\n", L, tokensGenerated);
        }
    }
    auto end = std::chrono::high_resolution_clock::now();
    std::chrono::duration<double> elapsed = end - start;
    printf("Generation took %f ms\n", elapsed.count() * 1000);
    printf("\n========================================\n");
    printf("Generation complete. Generated %d new tokens.\n", tokensGenerated);
    printf("Final sequence length: %d tokens\n", L);
    printf("========================================\n\n");
    printf("=== Final Generated Sequence ===\n");
    for (int i = 0; i < L; i++) print_escaped(vocabGetToken(seqTokenIndices[i]));
    printf("\n================================\n");
    return 0;
}
