// A main() shaped like the reference's (main.cu:177-226), built only against the replacement headers:
// allocateMemory -> loadModel | initializeRandomWeights -> loadVocab -> runInferenceLoop.
// usage: dropin_main <config 1..5 | 0 = reference defaults> <vocab.json> <stories.json> <story index> <context %> [model.bin]
//        [fast | verbose | interactive]   (fast: skipUserInput, quiet; verbose: skipUserInput + top-10 blocks;
//        interactive: verbose, one line of stdin per token, 'q' stops)  [maxL override]
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "mini_llm_reference_api.h"

int main(int argc, char** argv) {
    if (argc < 6) { printf("usage: %s cfg vocab stories index percent [model.bin]\n", argv[0]); return 2; }
    const int cfg = atoi(argv[1]);
    if (cfg > 0) {
        mlh_hparams hp;
        if (!mll_hparams_config(cfg, &hp)) return 2;
        if (argc > 8) hp.maxL = atoi(argv[8]);
        mllSetNetworkMeta(&hp);
    }
    allocateMemory(true);
    if (!mllDeviceContext()) return 3;
    if (argc > 6) { if (!loadModelFile(argv[6])) return 4; }
    else initializeRandomWeights(0.02f);
    if (!loadVocab(argv[2])) return 5;
    const char* mode = argc > 7 ? argv[7] : "fast";
    const bool verbose = mode[0] == 'v' || mode[0] == 'i';
    const bool skipUserInput = mode[0] != 'i';
    const int rc = runInferenceLoop(argv[3], atoi(argv[4]), atoi(argv[5]), skipUserInput, verbose);
    printf("ids:");
    const int maxL = mllGetNetworkMeta()->maxL;
    for (int i = 0; i < maxL; i++) printf(" %d", seqTokenIndices[i]);
    printf("\n");
    mllShutdown();
    return rc;
}
