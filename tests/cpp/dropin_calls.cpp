// Calls runInference(L) the way the reference's callers do -- on a grown, an unchanged, an edited and a
// shortened seqTokenIndices -- and runInferenceAllPositions, through the reference-named surface only, and
// writes what each call leaves on the device to <outdir>/<name>.f32 (raw floats) plus the token lists to
// <outdir>/tokens.txt, for the test to compare with the oracle.
// usage: dropin_calls <config> <vocab.json> <stories.json> <model.bin> <outdir>
#include <stdio.h>
#include <stdlib.h>

#include <string>
#include <vector>

#include "mini_llm_reference_api.h"

static std::string g_out;
static FILE* g_tok;

static int dump(const char* name, const float* data, size_t n) {
    FILE* f = fopen((g_out + "/" + name + ".f32").c_str(), "wb");
    if (!f) return 1;
    const size_t w = fwrite(data, sizeof(float), n, f);
    fclose(f);
    return w == n ? 0 : 1;
}

// runInference(L), then the last position's logits and probabilities as the token loop reads them.
static int run_and_dump(const char* name, int L) {
    if (runInference(L)) { printf("runInference(%d) failed at %s\n", L, name); return 1; }
    const int V = mllGetNetworkMeta()->vocabSize;
    std::vector<float> lg(V), pr(V);
    if (mlh_read_logits(mllDeviceContext(), 0, lg.data()) || mlh_read_probs(mllDeviceContext(), 0, pr.data())) return 1;
    TokenProb top[10];
    if (mll_top_k(mllDeviceContext(), 0, 10, top) != 10) return 1;
    fprintf(g_tok, "%s", name);
    for (int i = 0; i < L; i++) fprintf(g_tok, " %d", seqTokenIndices[i]);
    fprintf(g_tok, "\n%s_top", name);
    for (int i = 0; i < 10; i++) fprintf(g_tok, " %d", top[i].tokenIdx);
    fprintf(g_tok, "\n");
    return dump((std::string(name) + "_logits").c_str(), lg.data(), V) | dump((std::string(name) + "_probs").c_str(), pr.data(), V);
}

int main(int argc, char** argv) {
    if (argc < 6) { printf("usage: %s cfg vocab stories model.bin outdir\n", argv[0]); return 2; }
    mlh_hparams hp;
    if (!mll_hparams_config(atoi(argv[1]), &hp)) return 2;
    mllSetNetworkMeta(&hp);
    allocateMemory(true);
    if (!mllDeviceContext()) return 3;
    if (!loadModelFile(argv[4])) return 4;
    if (!loadVocab(argv[2])) return 5;
    g_out = argv[5];
    g_tok = fopen((g_out + "/tokens.txt").c_str(), "w");
    if (!g_tok) return 6;
    int L = loadStoryContext(argv[3], 0, 50);
    if (L < 12) return 7;
    int rc = run_and_dump("first", L);             // nothing cached: the whole context
    seqTokenIndices[L] = seqTokenIndices[2];
    seqTokenIndices[L + 1] = seqTokenIndices[5];
    rc |= run_and_dump("grown", L + 2);            // the cached prefix stays, two new positions are run
    rc |= run_and_dump("unchanged", L + 2);        // same tokens again: rebuilt from the start
    seqTokenIndices[3] = seqTokenIndices[7];
    rc |= run_and_dump("edited", L + 2);           // an early token changed: the cache is thrown away
    rc |= run_and_dump("shorter", L - 5);          // a prefix of what is cached: rebuilt
    seqTokenIndices[L - 5] = seqTokenIndices[0];
    rc |= run_and_dump("regrown", L - 4);          // and grown again by one from there
    const int V = hp.vocabSize;
    std::vector<float> probs((size_t)V * L);
    float loss = -1.0f;
    if (runInferenceAllPositions(L, probs.data(), &loss)) rc |= 1;
    fprintf(g_tok, "allpos");
    for (int i = 0; i < L; i++) fprintf(g_tok, " %d", seqTokenIndices[i]);
    fprintf(g_tok, "\nloss %.9g\n", loss);
    rc |= dump("allpos_probs", probs.data(), probs.size());
    rc |= run_and_dump("after_allpos", L + 1);     // the all-position call leaves L tokens cached: one more is run
    fclose(g_tok);
    mllShutdown();
    return rc;
}
