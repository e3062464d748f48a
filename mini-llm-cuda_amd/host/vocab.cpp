// vocab.json tokenizer and the tokenised-story prompt loader.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>
#include <vector>

#include "json.h"
#include "mini_llm_host.h"

using mll::Json;

#define VOCAB_HASH_SIZE 20011 // load_model.cu:138

struct mll_vocab {
    std::vector<char*> tokens;             // index -> string (NULL where the entry was not a string)
    std::vector<std::vector<int>> buckets; // chained hash table, newest entry first (load_model.cu:163-171)
};

// DJB2 (hash*33 + c), characters read through plain `char` into an int as
// load_model.cu:153-160 does, so bytes >= 0x80 enter sign-extended.
extern "C" unsigned int mll_hash_token(const char* str) {
    unsigned int hash = 5381;
    int c;
    while ((c = *str++)) hash = ((hash << 5) + hash) + (unsigned int)c;
    return hash % VOCAB_HASH_SIZE;
}

static bool read_file(const char* path, std::string& out) {
    FILE* f = fopen(path, "rb");
    if (!f) return false;
    fseek(f, 0, SEEK_END);
    long n = ftell(f);
    fseek(f, 0, SEEK_SET);
    out.resize(n > 0 ? (size_t)n : 0);
    size_t got = out.empty() ? 0 : fread(&out[0], 1, out.size(), f);
    fclose(f);
    out.resize(got);
    return true;
}

extern "C" mll_vocab* mll_vocab_load(const char* path, int expectSize) {
    printf("--- Attempting to load vocabulary from %s... ---\n", path ? path : "(null)");
    std::string text;
    if (!path || !read_file(path, text)) {
        printf("Error: Vocabulary file not found at '%s'\n", path ? path : "(null)");
        return nullptr;
    }
    Json root;
    std::string err;
    if (!mll::parseJson(text.data(), text.size(), root, err)) {
        printf("Error: Failed to parse vocabulary JSON.\n");
        return nullptr;
    }
    if (!root.isArray()) {
        printf("Error: Vocabulary JSON is not an array.\n");
        return nullptr;
    }
    const int arraySize = (int)root.arr.size();
    const int size = expectSize > 0 ? expectSize : arraySize;
    if (arraySize != size) // load_model.cu:238-241: a mismatch only warns
        printf("Warning: Vocabulary size (%d) differs from expected vocabSize (%d)\n", arraySize, size);
    mll_vocab* v = new mll_vocab();
    v->tokens.assign(size, nullptr);
    v->buckets.resize(VOCAB_HASH_SIZE);
    int loaded = 0;
    for (int i = 0; i < arraySize && i < size; i++) {
        const Json& item = root.arr[i];
        if (!item.isString()) continue;
        // cJSON hands out C strings: an embedded NUL ends the token there.
        const size_t len = strlen(item.str.c_str());
        v->tokens[i] = (char*)malloc(len + 1);
        memcpy(v->tokens[i], item.str.c_str(), len + 1);
        std::vector<int>& b = v->buckets[mll_hash_token(v->tokens[i])];
        b.insert(b.begin(), i); // chain at front
        loaded++;
    }
    printf("Loaded %d vocabulary tokens.\n--- Successfully loaded vocabulary. ---\n\n", loaded);
    return v;
}

extern "C" void mll_vocab_free(mll_vocab* v) {
    if (!v) return;
    for (char* t : v->tokens) free(t);
    delete v;
}

extern "C" int mll_vocab_size(const mll_vocab* v) { return v ? (int)v->tokens.size() : 0; }

extern "C" const char* mll_vocab_token(const mll_vocab* v, int index) {
    if (!v || index < 0 || index >= (int)v->tokens.size()) return nullptr;
    return v->tokens[index];
}

extern "C" int mll_vocab_lookup(const mll_vocab* v, const char* token) {
    if (!v || !token) return -1;
    for (int idx : v->buckets[mll_hash_token(token)])
        if (strcmp(v->tokens[idx], token) == 0) return idx;
    return -1;
}

static void print_token(const char* t) {
    if (strcmp(t, "\n") == 0) printf("[\\n]");
    else if (strcmp(t, "\t") == 0) printf("[\\t]");
    else printf("%s", t);
}

// main.cu:45-175
extern "C" int mll_load_story_context(const char* storiesPath, int storyIndex, int percentage,
                                      const mll_vocab* v, int maxL_, int32_t* out) {
    printf("--- Loading story context from %s ---\n", storiesPath ? storiesPath : "(null)");
    printf("Story index: %d, Context percentage: %d%%\n", storyIndex, percentage);
    std::string text;
    if (!storiesPath || !read_file(storiesPath, text)) {
        printf("Error: Stories file not found at '%s'\n", storiesPath ? storiesPath : "(null)");
        return 0;
    }
    Json root;
    std::string err;
    if (!mll::parseJson(text.data(), text.size(), root, err)) { printf("Error: Failed to parse stories JSON.\n"); return 0; }
    if (!root.isArray()) { printf("Error: Stories JSON is not an array.\n"); return 0; }
    const int numStories = (int)root.arr.size();
    if (storyIndex < 0 || storyIndex >= numStories) {
        printf("Error: Story index %d out of range (0-%d).\n", storyIndex, numStories - 1);
        return 0;
    }
    const Json& story = root.arr[storyIndex];
    if (!story.isArray()) { printf("Error: Story at index %d is not an array.\n", storyIndex); return 0; }
    const int totalTokens = (int)story.arr.size();
    if (totalTokens == 0) { printf("Error: Story at index %d has no tokens.\n", storyIndex); return 0; }
    int contextLength = (int)(((long long)totalTokens * percentage) / 100); // main.cu:114-119
    if (contextLength < 1) contextLength = 1;
    if (contextLength > maxL_ + 1) {
        printf("Warning: Context length %d exceeds max capacity (maxL+1=%d), truncating.\n", contextLength, maxL_ + 1);
        contextLength = maxL_ + 1;
    }
    printf("Story has %d tokens, using %d tokens as context.\n\n=== Story Context ===\n", totalTokens, contextLength);
    bool ok = true;
    for (int i = 0; i < contextLength; i++) {
        const Json& item = story.arr[i];
        if (!item.isString()) { printf("Error: Token at position %d is not a string.\n", i); ok = false; break; }
        const int idx = mll_vocab_lookup(v, item.str.c_str());
        if (idx < 0) { printf("Error: Token '%s' not found in vocabulary.\n", item.str.c_str()); ok = false; break; }
        out[i] = idx;
        print_token(item.str.c_str());
    }
    printf("\n=====================\n\n");
    if (!ok) return 0;
    printf("Set %d context tokens in seqTokenIndices (story length L=%d).\n", contextLength, contextLength);
    printf("--- Story context loaded successfully. ---\n\n");
    return contextLength;
}

// loadStoriesFromFile (training_orchestrator.cu:103-273): every story of a file into one slab of
// maxL+1 ids per story, padded with the padding token; rightEnd[i] = (tokens loaded) - 2, the last
// position whose next token is known.  Stories that are not arrays, are empty, hold fewer than two
// tokens, a non-string or a token outside the vocabulary are skipped with the reference's warnings.
extern "C" int mll_load_stories(const char* filePath, const mll_vocab* v, int maxL_, int maxStories, int32_t* tokens,
                                int32_t* rightEnd) {
    const int perStory = maxL_ + 1; // TOKENS_PER_STORY, training_orchestrator.h:9
    printf("--- Loading stories from %s ---\n", filePath ? filePath : "(null)");
    std::string text;
    if (!filePath || !read_file(filePath, text)) {
        printf("Error: Stories file not found at '%s'\n", filePath ? filePath : "(null)");
        return -1;
    }
    if (!tokens || !rightEnd || maxStories < 0 || maxL_ < 1) return -1;
    Json root;
    std::string err;
    if (!mll::parseJson(text.data(), text.size(), root, err)) { printf("Error: Failed to parse stories JSON.\n"); return -1; }
    if (!root.isArray()) { printf("Error: Stories JSON is not an array.\n"); return -1; }
    int numStories = (int)root.arr.size();
    if (numStories == 0) { printf("Warning: Stories file is empty.\n"); return 0; }
    if (numStories > maxStories) {
        printf("Warning: File contains %d stories, truncating to %d.\n", numStories, maxStories);
        numStories = maxStories;
    }
    printf("Processing %d stories...\n", numStories);
    int loaded = 0;
    for (int s = 0; s < numStories; s++) {
        const Json& story = root.arr[s];
        if (!story.isArray()) { printf("Warning: Story at index %d is not an array, skipping.\n", s); continue; }
        const int count = (int)story.arr.size();
        if (count == 0) { printf("Warning: Story at index %d has no tokens, skipping.\n", s); continue; }
        const int toLoad = count > perStory ? perStory : count;
        if (toLoad - 2 < 0) { printf("Warning: Story at index %d has fewer than 2 tokens, skipping.\n", s); continue; }
        int32_t* slot = tokens + (size_t)loaded * perStory;
        bool bad = false;
        for (int pos = 0; pos < toLoad; pos++) {
            const Json& item = story.arr[pos];
            if (!item.isString()) {
                printf("Warning: Token at position %d in story %d is not a string.\n", pos, s);
                bad = true;
                break;
            }
            const int idx = mll_vocab_lookup(v, item.str.c_str());
            if (idx < 0) {
                printf("Warning: Token '%s' not found in vocabulary (story %d, pos %d).\n", item.str.c_str(), s, pos);
                bad = true;
                break;
            }
            slot[pos] = idx;
        }
        if (bad) continue; // the slot is reused by the next story
        for (int pos = toLoad; pos < perStory; pos++) slot[pos] = MLL_PADDING_TOKEN_INDEX;
        rightEnd[loaded] = toLoad - 2;
        loaded++;
    }
    printf("Successfully processed %d stories (out of %d in file).\n", loaded, numStories);
    return loaded;
}
