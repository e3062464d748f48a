// Host-side model: hyper-parameter presets, seeded weight generator, model.bin
// reader and writer, upload to the device layer.
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>
#include <vector>

#include "json.h"
#include "mini_llm_host.h"

using mll::Json;

struct mll_model {
    mlh_hparams hp;
    std::vector<float> E, gF;
    std::vector<std::vector<std::vector<float>>> t; // [layer][tensor id] -> data (empty: absent)
};

// ---------------------------------------------------------------------------
// hyper-parameters
// ---------------------------------------------------------------------------
extern "C" void mll_hparams_reference_defaults(mlh_hparams* hp) { // network_meta.h:3-20
    memset(hp, 0, sizeof(*hp));
    hp->dim = 768; hp->attnHeads = 6; hp->headDim = 128; hp->ropeDenomBase = 10000.0f;
    hp->ffnDim = 3072; hp->transformers = 16; hp->maxL = 1280; hp->vocabSize = 20160;
    hp->qkRmsNorm = 1; hp->queryGating = 1;
    hp->weightDtype = MLH_DTYPE_F32; hp->maxSeqs = 1;
}

extern "C" void mll_set_layer_pattern(mlh_hparams* hp, int gdnPerAttn) {
    for (int t = 0; t < MLH_MAX_LAYERS; t++) hp->layerKinds[t] = MLH_KIND_ATTENTION;
    if (gdnPerAttn <= 0) return;
    for (int a = 0; a < hp->transformers; a++) { // a = application order, file index = transformers-1-a
        const int file = hp->transformers - 1 - a;
        hp->layerKinds[file] = (a % (gdnPerAttn + 1) == gdnPerAttn) ? MLH_KIND_ATTENTION : MLH_KIND_GDN;
    }
}

extern "C" int mll_hparams_config(int config, mlh_hparams* hp) {
    memset(hp, 0, sizeof(*hp));
    hp->ropeDenomBase = 10000.0f;
    hp->weightDtype = MLH_DTYPE_F32;
    hp->maxSeqs = 1;
    switch (config) {
        case 1: // tiny Llama-style decoder: 16-token prompt + 128 greedy steps
            hp->dim = 256; hp->attnHeads = 4; hp->headDim = 64; hp->ffnDim = 704; hp->transformers = 4;
            hp->vocabSize = 4096; hp->maxL = 16 + 128;
            mll_set_layer_pattern(hp, 0);
            return 1;
        case 2: // batch-1 full-attention decoder: 64-token prompt + 512 steps, KV up to 576
            hp->dim = 768; hp->attnHeads = 12; hp->headDim = 64; hp->ffnDim = 2048; hp->transformers = 12;
            hp->vocabSize = 8192; hp->maxL = 576;
            mll_set_layer_pattern(hp, 0);
            return 1;
        case 3: // hybrid 3 GDN : 1 attention, PLE 64: 128-token prompt + 1024 steps
        case 4: // the same model with 64 sequences, KV up to 2048 each
            hp->dim = 768; hp->attnHeads = 12; hp->headDim = 64; hp->ffnDim = 2048; hp->transformers = 12;
            hp->vocabSize = 8192; hp->gdnHeads = 12; hp->gdnDk = 64; hp->gdnDv = 64; hp->pleDim = 64;
            hp->maxL = config == 3 ? 128 + 1024 : 2048;
            hp->maxSeqs = config == 3 ? 1 : 64;
            mll_set_layer_pattern(hp, 3);
            return 1;
        case 5: // larger bf16 model: 8 x 2048-token prompts + 128 decode steps
            hp->dim = 2048; hp->attnHeads = 16; hp->headDim = 128; hp->ffnDim = 5632; hp->transformers = 24;
            hp->vocabSize = 32000; hp->gdnHeads = 16; hp->gdnDk = 128; hp->gdnDv = 128; hp->pleDim = 64;
            hp->maxL = 2048 + 128; hp->maxSeqs = 8; hp->weightDtype = MLH_DTYPE_BF16;
            mll_set_layer_pattern(hp, 3);
            return 1;
        default: return 0;
    }
}

// inference.cu:364-374, statement for statement (float powf/cosf/sinf, int * float product).
extern "C" void mll_rope_table(float* tab, int maxL_, int headDim_, float base) {
    const int numPairs = headDim_ / 2;
    for (int colIndex = 0; colIndex < maxL_; colIndex++) {
        const size_t colOffset = (size_t)colIndex * headDim_;
        for (int pairIndex = 0; pairIndex < numPairs; pairIndex++) {
            float theta = colIndex * powf(base, (-2.0f * pairIndex / headDim_));
            tab[colOffset + pairIndex * 2] = cosf(theta);
            tab[colOffset + pairIndex * 2 + 1] = sinf(theta);
        }
    }
}

// ---------------------------------------------------------------------------
// tensor inventory
// ---------------------------------------------------------------------------
struct TensorInfo {
    int id;
    const char* key; // model.bin header key
    int rows, cols;  // cols == 0: 1-D tensor of `rows` elements
};

// Per-block tensors in the read order of load_model.cu:411-450, then the
// extensions.  Tensors that are not part of this block are left out.
static std::vector<TensorInfo> block_tensors(const mlh_hparams& hp, int layer) {
    const bool attn = hp.layerKinds[layer] == MLH_KIND_ATTENTION;
    const int d = hp.dim, F = hp.ffnDim;
    const int qk = attn ? d : hp.gdnHeads * hp.gdnDk, vv = attn ? d : hp.gdnHeads * hp.gdnDv;
    std::vector<TensorInfo> v = {
        {MLH_T_RMS_GAMMA, "rmsGamma", d, 0},
        {MLH_T_QUERY, "queryWeights", qk, d},
        {MLH_T_KEY, "keyWeights", qk, d},
        {MLH_T_VALUE, "valueWeights", vv, d},
        {MLH_T_OUTPUT_PROJ, "outputProjectionWeights", d, vv},
        {MLH_T_RMS_GAMMA2, "rmsGamma2", d, 0},
        {MLH_T_FFN_1A, "feedForwardWeights1A", F, d},
        {MLH_T_FFN_1B, "feedForwardWeights1B", F, d},
        {MLH_T_FFN_2, "feedForwardWeights2", d, F},
    };
    if (attn && hp.qkRmsNorm) {
        v.push_back({MLH_T_QUERY_RMS_GAMMA, "queryRMSGamma", d, 0});
        v.push_back({MLH_T_KEY_RMS_GAMMA, "keyRMSGamma", d, 0});
    }
    if (attn && hp.queryGating) v.push_back({MLH_T_GATED_QUERY, "gatedQueryWeights", d, d});
    if (!attn) {
        v.push_back({MLH_T_GDN_ALPHA_W, "gdnAlphaWeights", hp.gdnHeads, d});
        v.push_back({MLH_T_GDN_ALPHA_B, "gdnAlphaBias", hp.gdnHeads, 0});
        v.push_back({MLH_T_GDN_BETA_W, "gdnBetaWeights", hp.gdnHeads, d});
        v.push_back({MLH_T_GDN_BETA_B, "gdnBetaBias", hp.gdnHeads, 0});
    }
    if (hp.pleDim > 0) {
        v.push_back({MLH_T_PLE_TABLE, "perLayerEmbeddings", hp.vocabSize, hp.pleDim});
        v.push_back({MLH_T_PLE_GATE, "pleGateWeights", hp.pleDim, d});
        v.push_back({MLH_T_PLE_UP, "pleUpWeights", d, hp.pleDim});
    }
    return v;
}

static size_t count_of(const TensorInfo& ti) { return (size_t)ti.rows * (ti.cols ? ti.cols : 1); }

extern "C" mll_model* mll_model_new(const mlh_hparams* hp) {
    if (!hp || hp->transformers <= 0 || hp->transformers > MLH_MAX_LAYERS || hp->dim <= 0 || hp->vocabSize <= 0)
        return nullptr;
    mll_model* m = new mll_model();
    m->hp = *hp;
    m->E.assign((size_t)hp->vocabSize * hp->dim, 0.f);
    m->gF.assign(hp->dim, 0.f);
    m->t.resize(hp->transformers);
    for (int l = 0; l < hp->transformers; l++) {
        m->t[l].resize(MLH_T_COUNT);
        for (const TensorInfo& ti : block_tensors(*hp, l)) m->t[l][ti.id].assign(count_of(ti), 0.f);
    }
    return m;
}

extern "C" void mll_model_free(mll_model* m) { delete m; }
extern "C" const mlh_hparams* mll_model_hparams(const mll_model* m) { return m ? &m->hp : nullptr; }

extern "C" float* mll_model_tensor(mll_model* m, int layer, int id, int* rows, int* cols) {
    if (!m) return nullptr;
    if (id == MLH_T_TOKEN_EMBEDDINGS) {
        if (rows) *rows = m->hp.vocabSize;
        if (cols) *cols = m->hp.dim;
        return m->E.data();
    }
    if (id == MLH_T_FINAL_RMS_GAMMA) {
        if (rows) *rows = m->hp.dim;
        if (cols) *cols = 1;
        return m->gF.data();
    }
    if (layer < 0 || layer >= m->hp.transformers || id < 0 || id >= MLH_T_COUNT) return nullptr;
    for (const TensorInfo& ti : block_tensors(m->hp, layer))
        if (ti.id == id) {
            if (rows) *rows = ti.rows;
            if (cols) *cols = ti.cols ? ti.cols : 1;
            return m->t[layer][id].data();
        }
    return nullptr;
}

// ---------------------------------------------------------------------------
// counter-based generator
// ---------------------------------------------------------------------------
static inline uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    uint64_t z = x;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
static inline uint64_t stream_base(uint64_t seed, uint64_t streamKey) {
    return splitmix64(splitmix64(seed) ^ (streamKey * 0xD1342543DE82EF95ull));
}
static inline uint64_t tensor_key(int layer, int id) { return (uint64_t)(layer + 1) * 64 + (uint64_t)id; }

// Box-Muller on two 53-bit uniforms per pair of elements; float64 maths, cast to float at the end.
static void fill_normal(float* w, size_t n, uint64_t base, double std) {
    const double TWO_PI = 6.283185307179586476925286766559;
    const size_t pairs = (n + 1) / 2;
#pragma omp parallel for schedule(static) if (n > 65536)
    for (size_t p = 0; p < pairs; p++) {
        const uint64_t a = splitmix64(base + 2 * p), b = splitmix64(base + 2 * p + 1);
        const double u1 = (double)((a >> 11) + 1) * (1.0 / 9007199254740992.0);
        const double u2 = (double)(b >> 11) * (1.0 / 9007199254740992.0);
        const double r = sqrt(-2.0 * log(u1));
        w[2 * p] = (float)(std * r * cos(TWO_PI * u2));
        if (2 * p + 1 < n) w[2 * p + 1] = (float)(std * r * sin(TWO_PI * u2));
    }
}

static void fill_uniform(float* w, size_t n, uint64_t base, double range) {
#pragma omp parallel for schedule(static) if (n > 65536)
    for (size_t i = 0; i < n; i++) {
        const double u = (double)(splitmix64(base + i) >> 11) * (1.0 / 9007199254740992.0);
        w[i] = (float)((2.0 * u - 1.0) * range);
    }
}

static bool is_gain(int id) {
    return id == MLH_T_RMS_GAMMA || id == MLH_T_RMS_GAMMA2 || id == MLH_T_QUERY_RMS_GAMMA ||
           id == MLH_T_KEY_RMS_GAMMA || id == MLH_T_FINAL_RMS_GAMMA;
}

static void init_model(mll_model* m, uint64_t seed, double scale, bool normal) {
    auto fill = [&](float* w, size_t n, int layer, int id) {
        const uint64_t base = stream_base(seed, tensor_key(layer, id));
        if (is_gain(id)) { for (size_t i = 0; i < n; i++) w[i] = 1.0f; return; } // random_weights.cu:47-49,58-60
        if (id == MLH_T_GDN_ALPHA_B || id == MLH_T_GDN_BETA_B) { fill_normal(w, n, base, 1.0); return; }
        if (normal) fill_normal(w, n, base, scale);
        else fill_uniform(w, n, base, scale);
    };
    fill(m->E.data(), m->E.size(), -1, MLH_T_TOKEN_EMBEDDINGS);
    fill(m->gF.data(), m->gF.size(), -1, MLH_T_FINAL_RMS_GAMMA);
    for (int l = 0; l < m->hp.transformers; l++)
        for (int id = 0; id < MLH_T_COUNT; id++)
            if (!m->t[l][id].empty()) fill(m->t[l][id].data(), m->t[l][id].size(), l, id);
}

extern "C" void mll_model_init_normal(mll_model* m, uint64_t seed, float std) { if (m) init_model(m, seed, std, true); }
extern "C" void mll_model_init_uniform(mll_model* m, uint64_t seed, float range) { if (m) init_model(m, seed, range, false); }

extern "C" void mll_random_tokens(uint64_t seed, int stream, int vocab, int n, int32_t* out) {
    const uint64_t base = stream_base(seed, 0x7000ull + (uint64_t)stream);
    for (int i = 0; i < n; i++) out[i] = (int32_t)(splitmix64(base + (uint64_t)i) % (uint64_t)vocab);
}

// ---------------------------------------------------------------------------
// model.bin
// ---------------------------------------------------------------------------
static void set_err(char* err, int errLen, const std::string& msg) {
    if (err && errLen > 0) snprintf(err, (size_t)errLen, "%s", msg.c_str());
    printf("Error: %s\n", msg.c_str());
}

struct TensorMeta { // parseTensorMeta, load_model.cu:24-61
    int shape[4];
    int dims;
    int bytesPerElement;
    size_t numElements;
};

static bool parse_tensor_meta(const Json* obj, TensorMeta& tm, std::string& why) {
    if (!obj || !obj->isObject()) { why = "tensor entry is not an object"; return false; }
    const Json* shape = obj->get("shape");
    if (!shape || !shape->isArray()) { why = "missing shape"; return false; }
    tm.dims = (int)shape->arr.size();
    if (tm.dims > 4) tm.dims = 4;
    tm.numElements = 1;
    for (int i = 0; i < tm.dims; i++) {
        tm.shape[i] = shape->arr[i].isNumber() ? shape->arr[i].asInt() : 0;
        if (tm.shape[i] < 0) { why = "negative shape"; return false; }
        tm.numElements *= (size_t)tm.shape[i];
    }
    const Json* dt = obj->get("dtype");
    if (!dt || !dt->isString()) { why = "missing dtype"; return false; }
    if (dt->str == "float32") tm.bytesPerElement = 4;
    else if (dt->str == "float64") tm.bytesPerElement = 8;
    else { why = "Unsupported dtype: " + dt->str; return false; }
    return true;
}

// Reads one tensor at the running offset (readTensorColumnMajor, load_model.cu:65-116,
// minus its transpose: the file's row-major [out, in] order is what the device layer takes).
static bool read_tensor(FILE* f, size_t fileSize, size_t& offset, const TensorMeta& tm, size_t expect,
                        float* dest, std::string& why) {
    if (tm.dims < 1 || tm.dims > 2) { why = "Unsupported tensor dimension: " + std::to_string(tm.dims); return false; }
    if (tm.numElements != expect) {
        why = "tensor has " + std::to_string(tm.numElements) + " elements, hyper-parameters expect " + std::to_string(expect);
        return false;
    }
    const size_t bytes = tm.numElements * (size_t)tm.bytesPerElement;
    if (offset + bytes > fileSize) { why = "Attempting to read past buffer end."; return false; }
    if (fseek(f, (long)offset, SEEK_SET) != 0) { why = "seek failed"; return false; }
    if (tm.bytesPerElement == 4) {
        if (fread(dest, 4, tm.numElements, f) != tm.numElements) { why = "short read"; return false; }
    } else {
        std::vector<double> tmp(std::min<size_t>(tm.numElements, 1 << 20));
        size_t done = 0;
        while (done < tm.numElements) {
            const size_t n = std::min(tmp.size(), tm.numElements - done);
            if (fread(tmp.data(), 8, n, f) != n) { why = "short read"; return false; }
            for (size_t i = 0; i < n; i++) dest[done + i] = (float)tmp[i]; // float64 -> float32, load_model.cu:81-85
            done += n;
        }
    }
    offset += bytes;
    return true;
}

static int json_int(const Json* o, const char* key, int dflt) {
    const Json* v = o ? o->get(key) : nullptr;
    if (!v) return dflt;
    if (v->type == Json::Bool) return v->b ? 1 : 0;
    return v->isNumber() ? v->asInt() : dflt;
}

static bool hparams_from_header(const Json& root, mlh_hparams& hp) {
    const Json* nm = root.get("networkMeta");
    if (!nm || !nm->isObject()) return false;
    memset(&hp, 0, sizeof(hp));
    hp.dim = json_int(nm, "dim", 0); hp.attnHeads = json_int(nm, "attnHeads", 0);
    hp.headDim = json_int(nm, "headDim", 0); hp.ffnDim = json_int(nm, "ffnDim", 0);
    hp.transformers = json_int(nm, "transformers", 0); hp.maxL = json_int(nm, "maxL", 0);
    hp.vocabSize = json_int(nm, "vocabSize", 0);
    const Json* rb = nm->get("ropeDenomBase");
    hp.ropeDenomBase = rb && rb->isNumber() ? (float)rb->num : 10000.0f;
    hp.qkRmsNorm = json_int(nm, "CONFIG_QK_RMS_NORM", 0); hp.queryGating = json_int(nm, "CONFIG_QUERY_GATING", 0);
    hp.gdnHeads = json_int(nm, "gdnHeads", 0); hp.gdnDk = json_int(nm, "gdnDk", 0); hp.gdnDv = json_int(nm, "gdnDv", 0);
    hp.pleDim = json_int(nm, "pleDim", 0);
    hp.weightDtype = json_int(nm, "weightDtype", 0); hp.maxSeqs = json_int(nm, "maxSeqs", 1);
    const Json* lk = nm->get("layerKinds");
    if (lk && lk->isArray())
        for (size_t i = 0; i < lk->arr.size() && i < MLH_MAX_LAYERS; i++) hp.layerKinds[i] = lk->arr[i].asInt();
    return hp.dim > 0 && hp.transformers > 0 && hp.transformers <= MLH_MAX_LAYERS && hp.vocabSize > 0;
}

extern "C" mll_model* mll_model_load(const char* path, const mlh_hparams* hint, char* err, int errLen) {
    printf("\n--- Attempting to load model weights from %s... ---\n", path ? path : "(null)");
    if (!path) { set_err(err, errLen, "null path"); return nullptr; }
    FILE* f = fopen(path, "rb");
    if (!f) { set_err(err, errLen, std::string("Model file not found at '") + path + "'"); return nullptr; }
    fseek(f, 0, SEEK_END);
    const size_t fileSize = (size_t)ftell(f);
    fseek(f, 0, SEEK_SET);
    auto failf = [&](const std::string& msg) { set_err(err, errLen, msg); fclose(f); return (mll_model*)nullptr; };

    unsigned char lenBytes[8];
    if (fileSize < 8 || fread(lenBytes, 1, 8, f) != 8) return failf("Failed to read file.");
    uint64_t headerLength = 0; // little-endian u64, load_model.cu:320-324
    for (int i = 0; i < 8; i++) headerLength |= ((uint64_t)lenBytes[i]) << (i * 8);
    const size_t headerEnd = 8 + (size_t)headerLength;
    if (headerLength > fileSize || headerEnd > fileSize)
        return failf("Header length specified in file is larger than the file itself.");
    std::string header(headerLength, '\0');
    if (headerLength && fread(&header[0], 1, headerLength, f) != headerLength) return failf("Failed to read file.");
    size_t offset = headerEnd + (8 - headerEnd % 8) % 8; // load_model.cu:340-343
    printf("Header length: %llu bytes\nData starts at offset: %zu\n", (unsigned long long)headerLength, offset);

    Json root;
    std::string perr;
    if (!mll::parseJson(header.data(), header.size(), root, perr) || !root.isObject())
        return failf("Error parsing JSON header. " + perr);

    mlh_hparams hp;
    if (hint) hp = *hint;
    else if (!hparams_from_header(root, hp))
        return failf("header has no networkMeta object and no hyper-parameters were supplied");
    mll_model* m = mll_model_new(&hp);
    if (!m) return failf("bad hyper-parameters");
    auto failm = [&](const std::string& msg) { mll_model_free(m); return failf(msg); };

    TensorMeta tm;
    std::string why;
    const Json* emb = root.get("tokenEmbeddings");
    if (emb) {
        if (!parse_tensor_meta(emb, tm, why)) return failm("tokenEmbeddings: " + why);
        printf("Loading tokenEmbeddings: [%d x %d]\n", tm.shape[0], tm.dims > 1 ? tm.shape[1] : 1);
        if (tm.dims == 2 && (tm.shape[0] != hp.vocabSize || tm.shape[1] != hp.dim))
            return failm("tokenEmbeddings must be [vocabSize, dim] (a [dim, vocabSize] header is the transposed "
                         "layout save_model.cu writes, which loadModel does not read back)");
        if (!read_tensor(f, fileSize, offset, tm, m->E.size(), m->E.data(), why)) return failm("tokenEmbeddings: " + why);
    }
    const Json* fin = root.get("finalRMSNormGamma");
    if (fin) {
        if (!parse_tensor_meta(fin, tm, why)) return failm("finalRMSNormGamma: " + why);
        if (!read_tensor(f, fileSize, offset, tm, m->gF.size(), m->gF.data(), why)) return failm("finalRMSNormGamma: " + why);
    }
    const Json* blocks = root.get("transformerBlocks");
    if (blocks && blocks->isArray()) {
        const int nb = (int)blocks->arr.size();
        for (int b = 0; b < hp.transformers && b < nb; b++) {
            const Json& blk = blocks->arr[b];
            if (!blk.isObject()) return failm("Expected transformer block object.");
            for (const TensorInfo& ti : block_tensors(hp, b)) {
                const Json* w = blk.get(ti.key);
                if (!w) { // load_model.cu:436-438,463-465: warn, do not advance the offset
                    printf("Warning: Weight '%s' not found in block %d\n", ti.key, b);
                    continue;
                }
                if (!parse_tensor_meta(w, tm, why)) return failm(std::string(ti.key) + ": " + why);
                if (tm.dims == 2 && ti.cols && (tm.shape[0] != ti.rows || tm.shape[1] != ti.cols))
                    return failm(std::string(ti.key) + ": shape does not match the hyper-parameters");
                if (!read_tensor(f, fileSize, offset, tm, count_of(ti), m->t[b][ti.id].data(), why))
                    return failm(std::string(ti.key) + " (block " + std::to_string(b) + "): " + why);
            }
        }
    }
    fclose(f);
    printf("--- Successfully loaded and assigned weights from %s. ---\n\n", path);
    return m;
}

static Json tensor_entry(int rows, int cols, bool f64) {
    Json e;
    e.type = Json::Object;
    e.obj.emplace_back("shape", cols ? mll::jsonIntArray({rows, cols}) : mll::jsonIntArray({rows}));
    e.obj.emplace_back("dtype", mll::jsonString(f64 ? "float64" : "float32"));
    return e;
}

static bool write_floats(FILE* f, const float* p, size_t n, bool f64) {
    if (!f64) return fwrite(p, 4, n, f) == n;
    std::vector<double> tmp(std::min<size_t>(n, 1 << 20));
    size_t done = 0;
    while (done < n) {
        const size_t k = std::min(tmp.size(), n - done);
        for (size_t i = 0; i < k; i++) tmp[i] = (double)p[done + i];
        if (fwrite(tmp.data(), 8, k, f) != k) return false;
        done += k;
    }
    return true;
}

extern "C" int mll_model_save(const mll_model* m, const char* path, int float64) {
    if (!m || !path) return 0;
    const mlh_hparams& hp = m->hp;
    const bool f64 = float64 != 0;
    Json root;
    root.type = Json::Object;
    root.obj.emplace_back("tokenEmbeddings", tensor_entry(hp.vocabSize, hp.dim, f64));
    root.obj.emplace_back("finalRMSNormGamma", tensor_entry(hp.dim, 0, f64));
    Json blocks;
    blocks.type = Json::Array;
    for (int l = 0; l < hp.transformers; l++) {
        Json b;
        b.type = Json::Object;
        for (const TensorInfo& ti : block_tensors(hp, l)) b.obj.emplace_back(ti.key, tensor_entry(ti.rows, ti.cols, f64));
        blocks.arr.push_back(std::move(b));
    }
    root.obj.emplace_back("transformerBlocks", std::move(blocks));
    Json nm;
    nm.type = Json::Object;
    auto num = [&](const char* k, double v) { nm.obj.emplace_back(k, mll::jsonNumber(v)); };
    num("dim", hp.dim); num("attnHeads", hp.attnHeads); num("headDim", hp.headDim);
    num("ropeDenomBase", hp.ropeDenomBase); num("ffnDim", hp.ffnDim); num("transformers", hp.transformers);
    num("maxL", hp.maxL); num("vocabSize", hp.vocabSize);
    num("CONFIG_QK_RMS_NORM", hp.qkRmsNorm); num("CONFIG_QUERY_GATING", hp.queryGating);
    num("gdnHeads", hp.gdnHeads); num("gdnDk", hp.gdnDk); num("gdnDv", hp.gdnDv); num("pleDim", hp.pleDim);
    num("weightDtype", hp.weightDtype); num("maxSeqs", hp.maxSeqs);
    nm.obj.emplace_back("layerKinds", mll::jsonIntArray(std::vector<int>(hp.layerKinds, hp.layerKinds + hp.transformers)));
    root.obj.emplace_back("networkMeta", std::move(nm));

    const std::string header = mll::dumpJson(root);
    FILE* f = fopen(path, "wb");
    if (!f) { printf("Error: cannot open '%s' for writing\n", path); return 0; }
    unsigned char lenBytes[8];
    for (int i = 0; i < 8; i++) lenBytes[i] = (unsigned char)(((uint64_t)header.size() >> (8 * i)) & 0xff);
    bool ok = fwrite(lenBytes, 1, 8, f) == 8 && fwrite(header.data(), 1, header.size(), f) == header.size();
    const size_t headerEnd = 8 + header.size();
    const size_t pad = (8 - headerEnd % 8) % 8;
    const unsigned char zeros[8] = {0};
    ok = ok && fwrite(zeros, 1, pad, f) == pad;
    ok = ok && write_floats(f, m->E.data(), m->E.size(), f64) && write_floats(f, m->gF.data(), m->gF.size(), f64);
    for (int l = 0; ok && l < hp.transformers; l++)
        for (const TensorInfo& ti : block_tensors(hp, l))
            ok = ok && write_floats(f, m->t[l][ti.id].data(), m->t[l][ti.id].size(), f64);
    ok = (fclose(f) == 0) && ok;
    if (!ok) printf("Error: failed writing '%s'\n", path);
    return ok ? 1 : 0;
}

// ---------------------------------------------------------------------------
// upload
// ---------------------------------------------------------------------------
extern "C" int mll_model_upload(const mll_model* m, mlh_ctx* ctx) {
    if (!m || !ctx) return 0;
    const mlh_hparams& hp = m->hp;
    auto bad = [&](const char* what) {
        printf("Error: upload of %s failed: %s\n", what, mlh_last_error(ctx));
        return 0;
    };
    if (mlh_upload_tensor(ctx, 0, MLH_T_TOKEN_EMBEDDINGS, m->E.data(), hp.vocabSize, hp.dim)) return bad("tokenEmbeddings");
    if (mlh_upload_tensor(ctx, 0, MLH_T_FINAL_RMS_GAMMA, m->gF.data(), hp.dim, 1)) return bad("finalRMSNormGamma");
    for (int l = 0; l < hp.transformers; l++)
        for (const TensorInfo& ti : block_tensors(hp, l))
            if (mlh_upload_tensor(ctx, l, ti.id, m->t[l][ti.id].data(), ti.rows, ti.cols ? ti.cols : 1)) return bad(ti.key);
    std::vector<float> rope((size_t)hp.maxL * hp.headDim);
    mll_rope_table(rope.data(), hp.maxL, hp.headDim, hp.ropeDenomBase);
    if (mlh_upload_rope_table(ctx, rope.data(), (int)rope.size())) return bad("RoPE table");
    if (mlh_finalize(ctx)) return bad("finalize");
    return 1;
}
