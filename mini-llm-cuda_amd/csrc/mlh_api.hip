// C ABI of the device layer: context life cycle, weight upload, sequence state,
// decode/prefill entry points, hipGraph capture and measurement helpers.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>

#include "mlh_internal.h"

static thread_local std::string g_create_error;

void mlh_set_thread_error(const std::string& msg) { g_create_error = msg; }

extern "C" const char* mlh_last_error(const mlh_ctx* ctx) {
    return ctx ? ctx->err.c_str() : g_create_error.c_str();
}

extern "C" int mlh_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

extern "C" int mlh_kv_page_size(void) { return MLH_KV_PAGE; }

static const char* const kKernelNames[MLH_K_COUNT] = {
    "k_phaseA", "k_attn", "k_oproj", "k_ffn13", "k_down", "k_lmhead", "k_gdn", "k_copy", "k_embed", "k_finish"};
extern "C" const char* mlh_kernel_name(int kernel) {
    return (kernel >= 0 && kernel < MLH_K_COUNT) ? kKernelNames[kernel] : "";
}

int mlh_dev_alloc_bytes(mlh_ctx* c, void** p, size_t bytes) {
    void* q = nullptr;
    MLH_CHECK(c, hipMalloc(&q, bytes));
    c->allocs.push_back(q);
    *p = q;
    return 0;
}

static int fail_create(const std::string& msg) {
    g_create_error = msg;
    return -1;
}

static std::string validate(const mlh_hparams& hp) {
    if (hp.dim <= 0 || hp.attnHeads <= 0 || hp.headDim <= 0 || hp.ffnDim <= 0 || hp.transformers <= 0 ||
        hp.maxL <= 0 || hp.vocabSize <= 0 || hp.maxSeqs <= 0)
        return "hyper-parameters must be positive";
    if (hp.transformers > MLH_MAX_LAYERS) return "too many layers";
    if (hp.attnHeads * hp.headDim != hp.dim) return "attnHeads * headDim must equal dim";
    if (hp.dim % 8 || hp.ffnDim % 8) return "dim and ffnDim must be multiples of 8";
    if (hp.pleDim < 0 || hp.pleDim % 8) return "pleDim must be a multiple of 8";
    if (hp.weightDtype != MLH_DTYPE_F32 && hp.weightDtype != MLH_DTYPE_BF16) return "unknown weightDtype";
    bool anyGdn = false, anyAttn = false;
    for (int t = 0; t < hp.transformers; t++) {
        if (hp.layerKinds[t] == MLH_KIND_GDN) anyGdn = true;
        else if (hp.layerKinds[t] == MLH_KIND_ATTENTION) anyAttn = true;
        else return "unknown layer kind";
    }
    if (anyAttn && hp.headDim != 64 && hp.headDim != 128) return "headDim must be 64 or 128";
    if (anyGdn) {
        if (!((hp.gdnDk == 64 && hp.gdnDv == 64) || (hp.gdnDk == 128 && hp.gdnDv == 128)))
            return "GDN needs dk = dv = 64 or 128";
        if (hp.gdnHeads <= 0) return "gdnHeads must be positive";
    }
    if ((size_t)hp.dim * 4 > 40 * 1024) return "dim too large for the LDS-staged GEMV (max 10240)";
    return "";
}

template <typename T>
static int dev_alloc(mlh_ctx* c, T** p, size_t count, bool zero = true) {
    void* q = nullptr;
    size_t bytes = std::max<size_t>(count * sizeof(T), 16);
    MLH_CHECK(c, hipMalloc(&q, bytes));
    c->allocs.push_back(q);
    if (zero) MLH_CHECK(c, hipMemset(q, 0, bytes));
    *p = (T*)q;
    return 0;
}

extern "C" void mlh_destroy(mlh_ctx* c) {
    if (!c) return;
    (void)hipSetDevice(c->device);
    if (c->stream) (void)hipStreamSynchronize(c->stream);
    for (int i = 0; i < 2; i++) if (c->graphExec[i]) (void)hipGraphExecDestroy(c->graphExec[i]);
    for (void* p : c->allocs) (void)hipFree(p);
    for (void* p : c->pfAllocs) (void)hipFree(p);
    for (void* p : c->mirrorAllocs) (void)hipFree(p);
    if (c->pfGdnWs) (void)hipFree(c->pfGdnWs);
    if (c->pfGdnG) (void)hipFree(c->pfGdnG);
    if (c->stream) (void)hipStreamDestroy(c->stream);
    delete c;
}

extern "C" int mlh_create(const mlh_hparams* hpIn, int device, mlh_ctx** out) {
    if (!hpIn || !out) return fail_create("null argument");
    *out = nullptr;
    std::string v = validate(*hpIn);
    if (!v.empty()) return fail_create(v);
    int ndev = mlh_device_count();
    if (ndev <= 0) return fail_create("no HIP device is visible: the MI355X path cannot run without a GPU");
    if (device < 0 || device >= ndev) return fail_create("device index out of range");
    if (hipSetDevice(device) != hipSuccess) return fail_create("hipSetDevice failed");
    if (mlh_gemm_device_init(device)) return -2; // address of this device's static workspace (mlh_gemm_device); message already set

    mlh_ctx* c = new mlh_ctx();
    c->hp = *hpIn;
    c->device = device;
    const mlh_hparams& hp = c->hp;
    c->wbytes = hp.weightDtype == MLH_DTYPE_BF16 ? 2 : 4;
    int rc = 0;
    auto bail = [&](int code) {
        g_create_error = c->err;
        mlh_destroy(c);
        return code;
    };
    if (hipStreamCreate(&c->stream) != hipSuccess) {
        c->err = "hipStreamCreate failed";
        return bail(-2);
    }

    const int d = hp.dim, F = hp.ffnDim, V = hp.vocabSize, pl = hp.pleDim, S = hp.maxSeqs;
    c->pagesPerSeq = (hp.maxL + MLH_KV_PAGE - 1) / MLH_KV_PAGE;
    // batch-1..few: split the keys over several workgroups per head; many
    // sequences already fill the chip, so one workgroup walks all its tiles.
    const int wgKeys = (hp.headDim <= 64 ? 4 : 2) * 64;
    c->nsplit = S >= 16 ? 1 : std::max(1, (hp.maxL + wgKeys - 1) / wgKeys);
    if (c->nsplit > 8) c->nsplit = 8;
    c->layers.resize(hp.transformers);
    c->have.assign(hp.transformers, std::vector<char>(MLH_T_COUNT, 0));
    char* tmp;
    if ((rc = dev_alloc(c, &tmp, (size_t)V * d * c->wbytes))) return bail(rc);
    c->E = tmp;
    if ((rc = dev_alloc(c, &c->gF, d))) return bail(rc);
    if ((rc = dev_alloc(c, &c->rope, (size_t)hp.maxL * hp.headDim))) return bail(rc);

    const size_t poolFloats = (size_t)S * c->pagesPerSeq * MLH_KV_PAGE * d;
    for (int t = 0; t < hp.transformers; t++) {
        LayerDev& L = c->layers[t];
        memset(&L, 0, sizeof(L));
        L.kind = hp.layerKinds[t];
        int r = 0;
        if (L.kind == MLH_KIND_ATTENTION) {
            L.offK = d; L.offV = 2 * d; r = 3 * d;
            if (hp.queryGating) { L.offG = r; r += d; }
            L.ad = d;
        } else {
            const int qk = hp.gdnHeads * hp.gdnDk, vv = hp.gdnHeads * hp.gdnDv;
            L.offK = qk; L.offV = 2 * qk; r = 2 * qk + vv;
            L.ad = vv;
        }
        if (pl > 0) { L.offPle = r; r += pl; }
        if (L.kind == MLH_KIND_GDN) { L.offGa = r; r += hp.gdnHeads; L.offGb = r; r += hp.gdnHeads; }
        L.rowsA = r;
        c->maxRowsA = std::max(c->maxRowsA, r);
        c->maxAd = std::max(c->maxAd, L.ad);
        if (L.ad % 8) { c->err = "mixing width must be a multiple of 8"; return bail(-1); }
        char *wa, *wo, *w13, *w2, *pu = nullptr, *pt = nullptr;
        if ((rc = dev_alloc(c, &wa, (size_t)r * d * c->wbytes))) return bail(rc);
        if ((rc = dev_alloc(c, &wo, (size_t)d * L.ad * c->wbytes))) return bail(rc);
        if ((rc = dev_alloc(c, &w13, (size_t)2 * F * d * c->wbytes))) return bail(rc);
        if ((rc = dev_alloc(c, &w2, (size_t)d * F * c->wbytes))) return bail(rc);
        if (pl > 0) {
            if ((rc = dev_alloc(c, &pu, (size_t)d * pl * c->wbytes))) return bail(rc);
            if ((rc = dev_alloc(c, &pt, (size_t)V * pl * c->wbytes))) return bail(rc);
        }
        L.Wa = wa; L.Wo = wo; L.W13 = w13; L.W2 = w2; L.pleUp = pu; L.pleTable = pt;
        float *g1, *g2, *gq = nullptr, *gk = nullptr, *ba = nullptr, *bb = nullptr;
        if ((rc = dev_alloc(c, &g1, d)) || (rc = dev_alloc(c, &g2, d))) return bail(rc);
        if (L.kind == MLH_KIND_ATTENTION) {
            if (hp.qkRmsNorm && ((rc = dev_alloc(c, &gq, d)) || (rc = dev_alloc(c, &gk, d)))) return bail(rc);
            if ((rc = dev_alloc(c, &L.K, poolFloats)) || (rc = dev_alloc(c, &L.V, poolFloats))) return bail(rc);
        } else {
            if ((rc = dev_alloc(c, &ba, hp.gdnHeads)) || (rc = dev_alloc(c, &bb, hp.gdnHeads))) return bail(rc);
            if ((rc = dev_alloc(c, &L.S, (size_t)S * hp.gdnHeads * hp.gdnDk * hp.gdnDv))) return bail(rc);
        }
        L.g1 = g1; L.g2 = g2; L.gq = gq; L.gk = gk; L.gdnBa = ba; L.gdnBb = bb;
    }
    if ((size_t)std::max(c->maxAd + pl, F) * 4 > 48 * 1024) {
        c->err = "ffnDim / mixing width too large for the LDS-staged GEMV";
        return bail(-1);
    }

    c->amaxParts = (V + 15) / 16; // one partial per LM-head workgroup (16 rows each)
    c->outCapacity = hp.maxL;
    c->promptCapacity = hp.maxL;
    if ((rc = dev_alloc(c, &c->d_sidx, S)) || (rc = dev_alloc(c, &c->d_tok, S)) ||
        (rc = dev_alloc(c, &c->d_pos, S)) || (rc = dev_alloc(c, &c->d_pageTable, (size_t)S * c->pagesPerSeq)) ||
        (rc = dev_alloc(c, &c->d_outIds, (size_t)c->outCapacity * S)) || (rc = dev_alloc(c, &c->d_stepCounter, 1)) || (rc = dev_alloc(c, &c->d_next, S)) ||
        (rc = dev_alloc(c, &c->d_prompt, c->promptCapacity)) || (rc = dev_alloc(c, &c->x, (size_t)S * d)) ||
        (rc = dev_alloc(c, &c->qkv, (size_t)S * c->maxRowsA)) ||
        (rc = dev_alloc(c, &c->part, (size_t)S * c->nsplit * hp.attnHeads * (hp.headDim + 2))) ||
        (rc = dev_alloc(c, &c->mix, (size_t)S * c->maxAd)) || (rc = dev_alloc(c, &c->h1, (size_t)S * d)) ||
        (rc = dev_alloc(c, &c->u, (size_t)S * F)) || (rc = dev_alloc(c, &c->logits, (size_t)S * V)) ||
        (rc = dev_alloc(c, &c->probs, V)) || (rc = dev_alloc(c, &c->amaxVal, (size_t)S * c->amaxParts)) ||
        (rc = dev_alloc(c, &c->amaxIdx, (size_t)S * c->amaxParts)))
        return bail(rc);
    {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, device) != hipSuccess) { c->err = "hipGetDeviceProperties failed"; return bail(-2); }
        c->numCUs = prop.multiProcessorCount;
        c->coopLaunch = prop.cooperativeLaunch != 0;
    }
    if ((rc = dev_alloc(c, &c->d_layers, (size_t)hp.transformers)) || (rc = dev_alloc(c, &c->d_sync, 64 * 24)) ||
        (rc = dev_alloc(c, &c->pamaxVal, (size_t)c->numCUs)) || (rc = dev_alloc(c, &c->pamaxIdx, (size_t)c->numCUs)) ||
        (rc = dev_alloc(c, &c->kvPart, (size_t)hp.attnHeads * c->pagesPerSeq * (hp.headDim + 2))))
        return bail(rc);
    c->xcdWords = mlh_xcd_words(c);
    if ((rc = dev_alloc(c, &c->xcdBuf, c->xcdWords))) return bail(rc);
    if (hipMemset(c->xcdBuf, 0, c->xcdWords * 8) != hipSuccess || hipMemset(c->d_sync, 0, 64 * 24 * 4) != hipSuccess) {
        c->err = "clearing the exchange words failed";
        return bail(-2);
    }
    c->persistCooperative = getenv("MLH_PERSIST_COOPERATIVE") != nullptr; // like the knobs below: the environment is read here only
    if (getenv("MLH_PERSIST_TIMING") && (rc = dev_alloc(c, &c->d_timing, (size_t)16 * (hp.transformers + 1) + 4 * 256))) return bail(rc);
    c->copyBytes = (size_t)256 << 20; // calibration copy of MLH_K_COPY: the two buffers are allocated on its first use
    {   // tuning knobs of the XCD-rank kernel: read once, here
        auto knob = [](const char* name, int dflt, int lo, int hi) {
            const char* e = getenv(name);
            return e ? std::max(lo, std::min(hi, atoi(e))) : dflt;
        };
        c->xcdWide = knob("MLH_XCD_WIDE", 1, 0, 1);
        c->xcdNapRound = knob("MLH_XCD_NAP_ROUND", 0, 0, 400);
        static const char* names[5] = {"MLH_XCD_NAP_CROSS", "MLH_XCD_NAP_GATHER", "MLH_XCD_NAP_QKV", "MLH_XCD_NAP_U", "MLH_XCD_NAP_PART"};
        // Measured one at a time and in combination on the benchmark shapes: a short stay away from the FFN activations
        // and the softmax partials pays from dim 768 on (+0.6 %), and costs 2 % on the 256-wide model.
        const bool wideModel = hp.dim >= 512;
        const int dflt[5] = {44, 0, 0, wideModel ? 6 : 0, wideModel ? 16 : 0};
        for (int k = 0; k < 5; k++) c->xcdNap[k] = knob(names[k], dflt[k], 0, 400);
    }

    std::vector<int> pt((size_t)S * c->pagesPerSeq);
    for (size_t i = 0; i < pt.size(); i++) pt[i] = (int)i;
    if (hipMemcpy(c->d_pageTable, pt.data(), pt.size() * 4, hipMemcpyHostToDevice) != hipSuccess) {
        c->err = "page table upload failed";
        return bail(-2);
    }
    c->h_len.assign(S, 0);
    *out = c;
    return 0;
}

static void to_bf16(const float* src, bf16_t* dst, size_t n) {
    for (size_t i = 0; i < n; i++) {
        uint32_t u;
        memcpy(&u, &src[i], 4);
        if ((u & 0x7fffffffu) > 0x7f800000u) u |= 0x00400000u; // keep NaN quiet
        else u += 0x7fffu + ((u >> 16) & 1u);                  // round to nearest even
        dst[i] = (bf16_t)(u >> 16);
    }
}

// Copies a row-major [rows, cols] fp32 host matrix into a device matrix of the
// context's weight dtype, row i going to dst row (rowOff + i*rowStep).
static int upload_matrix(mlh_ctx* c, void* dst, int dstCols, int rowOff, int rowStep, const float* host,
                         int rows, int cols) {
    if (cols != dstCols) { c->err = "tensor column count does not match the hyper-parameters"; return -1; }
    const size_t wb = c->wbytes;
    const void* src = host;
    std::vector<bf16_t> tmp;
    if (c->hp.weightDtype == MLH_DTYPE_BF16) {
        tmp.resize((size_t)rows * cols);
        to_bf16(host, tmp.data(), tmp.size());
        src = tmp.data();
    }
    char* d0 = (char*)dst + (size_t)rowOff * dstCols * wb;
    MLH_CHECK(c, hipMemcpy2D(d0, (size_t)rowStep * dstCols * wb, src, (size_t)cols * wb, (size_t)cols * wb, rows,
                             hipMemcpyHostToDevice));
    return 0;
}

static int upload_vec(mlh_ctx* c, const float* dst, const float* host, int n, int expect) {
    if (n != expect) { c->err = "vector length does not match the hyper-parameters"; return -1; }
    MLH_CHECK(c, hipMemcpy((void*)dst, host, (size_t)n * 4, hipMemcpyHostToDevice));
    return 0;
}

extern "C" int mlh_upload_tensor(mlh_ctx* c, int layer, int id, const float* host, int rows, int cols) {
    if (!c) return -1;
    if (!host || rows <= 0 || cols <= 0) { c->err = "bad tensor argument"; return -1; }
    (void)hipSetDevice(c->device);
    const mlh_hparams& hp = c->hp;
    const int d = hp.dim, F = hp.ffnDim, V = hp.vocabSize, pl = hp.pleDim;
    c->finalized = false;
    int rc;
    if (id == MLH_T_TOKEN_EMBEDDINGS) {
        if (rows != V) { c->err = "tokenEmbeddings must be [vocabSize, dim]"; return -1; }
        if ((rc = upload_matrix(c, c->E, d, 0, 1, host, rows, cols))) return rc;
        c->haveE = true;
        return 0;
    }
    if (id == MLH_T_FINAL_RMS_GAMMA) {
        if ((rc = upload_vec(c, c->gF, host, rows * cols, d))) return rc;
        c->haveGF = true;
        return 0;
    }
    if (layer < 0 || layer >= hp.transformers) { c->err = "layer index out of range"; return -1; }
    if (id < MLH_T_RMS_GAMMA || id >= MLH_T_COUNT) { c->err = "unknown tensor id"; return -1; }
    LayerDev& L = c->layers[layer];
    const bool attn = L.kind == MLH_KIND_ATTENTION;
    const int qk = attn ? d : hp.gdnHeads * hp.gdnDk, vv = attn ? d : hp.gdnHeads * hp.gdnDv;
    auto rowsMustBe = [&](int r) {
        if (rows != r) { c->err = "tensor row count does not match the hyper-parameters"; return false; }
        return true;
    };
    rc = 0;
    switch (id) {
        case MLH_T_RMS_GAMMA: rc = upload_vec(c, L.g1, host, rows * cols, d); break;
        case MLH_T_RMS_GAMMA2: rc = upload_vec(c, L.g2, host, rows * cols, d); break;
        case MLH_T_QUERY: if (!rowsMustBe(qk)) return -1; rc = upload_matrix(c, (void*)L.Wa, d, 0, 1, host, rows, cols); break;
        case MLH_T_KEY: if (!rowsMustBe(qk)) return -1; rc = upload_matrix(c, (void*)L.Wa, d, L.offK, 1, host, rows, cols); break;
        case MLH_T_VALUE: if (!rowsMustBe(vv)) return -1; rc = upload_matrix(c, (void*)L.Wa, d, L.offV, 1, host, rows, cols); break;
        case MLH_T_OUTPUT_PROJ: if (!rowsMustBe(d)) return -1; rc = upload_matrix(c, (void*)L.Wo, L.ad, 0, 1, host, rows, cols); break;
        case MLH_T_FFN_1A: if (!rowsMustBe(F)) return -1; rc = upload_matrix(c, (void*)L.W13, d, 0, 2, host, rows, cols); break;
        case MLH_T_FFN_1B: if (!rowsMustBe(F)) return -1; rc = upload_matrix(c, (void*)L.W13, d, 1, 2, host, rows, cols); break;
        case MLH_T_FFN_2: if (!rowsMustBe(d)) return -1; rc = upload_matrix(c, (void*)L.W2, F, 0, 1, host, rows, cols); break;
        case MLH_T_QUERY_RMS_GAMMA:
        case MLH_T_KEY_RMS_GAMMA:
            if (!attn || !hp.qkRmsNorm) { c->err = "Q/K RMS gains are not part of this layer"; return -1; }
            rc = upload_vec(c, id == MLH_T_QUERY_RMS_GAMMA ? L.gq : L.gk, host, rows * cols, d);
            break;
        case MLH_T_GATED_QUERY:
            if (!attn || !hp.queryGating) { c->err = "gated query weights are not part of this layer"; return -1; }
            if (!rowsMustBe(d)) return -1;
            rc = upload_matrix(c, (void*)L.Wa, d, L.offG, 1, host, rows, cols);
            break;
        case MLH_T_GDN_ALPHA_W:
        case MLH_T_GDN_BETA_W:
            if (attn) { c->err = "GDN gate weights given for an attention layer"; return -1; }
            if (!rowsMustBe(hp.gdnHeads)) return -1;
            rc = upload_matrix(c, (void*)L.Wa, d, id == MLH_T_GDN_ALPHA_W ? L.offGa : L.offGb, 1, host, rows, cols);
            break;
        case MLH_T_GDN_ALPHA_B:
        case MLH_T_GDN_BETA_B:
            if (attn) { c->err = "GDN gate bias given for an attention layer"; return -1; }
            rc = upload_vec(c, id == MLH_T_GDN_ALPHA_B ? L.gdnBa : L.gdnBb, host, rows * cols, hp.gdnHeads);
            break;
        case MLH_T_PLE_TABLE:
            if (pl <= 0) { c->err = "model has no per-layer embeddings"; return -1; }
            if (!rowsMustBe(V)) return -1;
            rc = upload_matrix(c, (void*)L.pleTable, pl, 0, 1, host, rows, cols);
            break;
        case MLH_T_PLE_GATE:
            if (pl <= 0) { c->err = "model has no per-layer embeddings"; return -1; }
            if (!rowsMustBe(pl)) return -1;
            rc = upload_matrix(c, (void*)L.Wa, d, L.offPle, 1, host, rows, cols);
            break;
        case MLH_T_PLE_UP:
            if (pl <= 0) { c->err = "model has no per-layer embeddings"; return -1; }
            if (!rowsMustBe(d)) return -1;
            rc = upload_matrix(c, (void*)L.pleUp, pl, 0, 1, host, rows, cols);
            break;
        default: c->err = "unknown tensor id"; return -1;
    }
    if (rc == 0) c->have[layer][id] = 1;
    return rc;
}

extern "C" int mlh_upload_rope_table(mlh_ctx* c, const float* tab, int n) {
    if (!c) return -1;
    if (!tab || n != c->hp.maxL * c->hp.headDim) { c->err = "RoPE table must be [maxL, headDim]"; return -1; }
    (void)hipSetDevice(c->device);
    MLH_CHECK(c, hipMemcpy(c->rope, tab, (size_t)n * 4, hipMemcpyHostToDevice));
    c->haveRope = true;
    return 0;
}

extern "C" int mlh_finalize(mlh_ctx* c) {
    if (!c) return -1;
    const mlh_hparams& hp = c->hp;
    if (!c->haveE || !c->haveGF || !c->haveRope) { c->err = "embeddings, final gain or RoPE table missing"; return -1; }
    for (int t = 0; t < hp.transformers; t++) {
        const bool attn = c->layers[t].kind == MLH_KIND_ATTENTION;
        std::vector<int> need = {MLH_T_RMS_GAMMA, MLH_T_QUERY, MLH_T_KEY, MLH_T_VALUE, MLH_T_OUTPUT_PROJ,
                                 MLH_T_RMS_GAMMA2, MLH_T_FFN_1A, MLH_T_FFN_1B, MLH_T_FFN_2};
        if (attn && hp.qkRmsNorm) { need.push_back(MLH_T_QUERY_RMS_GAMMA); need.push_back(MLH_T_KEY_RMS_GAMMA); }
        if (attn && hp.queryGating) need.push_back(MLH_T_GATED_QUERY);
        if (!attn) for (int id = MLH_T_GDN_ALPHA_W; id <= MLH_T_GDN_BETA_B; id++) need.push_back(id);
        if (hp.pleDim > 0) for (int id = MLH_T_PLE_TABLE; id <= MLH_T_PLE_UP; id++) need.push_back(id);
        for (int id : need)
            if (!c->have[t][id]) {
                c->err = "layer " + std::to_string(t) + ": tensor " + std::to_string(id) + " was not uploaded";
                return -1;
            }
    }
    (void)hipSetDevice(c->device);
    int rc = mlh_init_kernels(c);
    if (rc == 0) rc = mlh_init_prefill_kernels(c);
    if (rc == 0) rc = mlh_build_gemm_operands(c);
    if (rc) return rc;
    MLH_CHECK(c, hipMemcpy(c->d_layers, c->layers.data(), c->layers.size() * sizeof(LayerDev), hipMemcpyHostToDevice));
    // function attributes and occupancy of the single-launch decode kernels, here and not on every launch
    c->xcdPrepared = c->persistentPrepared = false;
    if (mlh_xcd_supported(c) && (rc = mlh_launch_xcd(c, 0))) return rc;
    if (mlh_persistent_supported(c) && mlh_launch_persistent(c, 0)) c->err.clear(); // a model too wide for it simply does not use it
    MLH_CHECK(c, hipDeviceSynchronize());
    c->finalized = true;
    return 0;
}

static int check_ready(mlh_ctx* c) {
    if (!c) return -1;
    if (!c->finalized) { c->err = "mlh_finalize has not succeeded on this context"; return -1; }
    (void)hipSetDevice(c->device);
    return 0;
}

extern "C" int mlh_reset(mlh_ctx* c, int seq) {
    if (!c) return -1;
    (void)hipSetDevice(c->device);
    const mlh_hparams& hp = c->hp;
    if (seq < -1 || seq >= hp.maxSeqs) { c->err = "sequence index out of range"; return -1; }
    const int s0 = seq < 0 ? 0 : seq, s1 = seq < 0 ? hp.maxSeqs : seq + 1;
    MLH_CHECK(c, hipStreamSynchronize(c->stream));
    MLH_CHECK(c, hipMemset(c->d_pos + s0, 0, (size_t)(s1 - s0) * 4));
    const size_t per = (size_t)hp.gdnHeads * hp.gdnDk * hp.gdnDv;
    for (int t = 0; t < hp.transformers; t++)
        if (c->layers[t].S) MLH_CHECK(c, hipMemset(c->layers[t].S + s0 * per, 0, (s1 - s0) * per * 4));
    for (int s = s0; s < s1; s++) c->h_len[s] = 0;
    return 0;
}

extern "C" int mlh_seq_len(mlh_ctx* c, int seq) {
    if (!c || seq < 0 || seq >= c->hp.maxSeqs) return -1;
    return c->h_len[seq];
}

extern "C" int mlh_max_len(const mlh_ctx* c) { return c ? c->hp.maxL : -1; }
extern "C" int mlh_vocab_size(const mlh_ctx* c) { return c ? c->hp.vocabSize : -1; }

extern "C" int mlh_greedy_token(mlh_ctx* c, int seq, int32_t* id) {
    if (!c) return -1;
    if (seq < 0 || seq >= c->hp.maxSeqs || !id) { c->err = "bad argument"; return -1; }
    (void)hipSetDevice(c->device);
    MLH_CHECK(c, hipStreamSynchronize(c->stream));
    MLH_CHECK(c, hipMemcpy(id, c->d_next + seq, 4, hipMemcpyDeviceToHost));
    return 0;
}

extern "C" int mlh_set_page_table(mlh_ctx* c, const int32_t* table, int n) {
    if (!c) return -1;
    const int total = c->hp.maxSeqs * c->pagesPerSeq;
    if (!table || n != total) { c->err = "page table must have maxSeqs * pagesPerSeq entries"; return -1; }
    std::vector<char> seen(total, 0);
    for (int i = 0; i < n; i++) {
        if (table[i] < 0 || table[i] >= total || seen[table[i]]) { c->err = "page table must be a permutation of the pool slots"; return -1; }
        seen[table[i]] = 1;
    }
    (void)hipSetDevice(c->device);
    MLH_CHECK(c, hipStreamSynchronize(c->stream));
    MLH_CHECK(c, hipMemcpy(c->d_pageTable, table, (size_t)n * 4, hipMemcpyHostToDevice));
    return 0;
}

static int set_slots(mlh_ctx* c, const int* seqs, int n) {
    bool identity = true;
    for (int i = 0; i < n; i++) identity = identity && seqs[i] == i;
    if (identity && c->identityNseq >= n) return 0;
    MLH_CHECK(c, hipMemcpyAsync(c->d_sidx, seqs, (size_t)n * 4, hipMemcpyHostToDevice, c->stream));
    MLH_CHECK(c, hipStreamSynchronize(c->stream));
    c->identityNseq = identity ? n : 0;
    return 0;
}

static int set_identity_slots(mlh_ctx* c, int nseq) {
    std::vector<int> id(nseq);
    for (int i = 0; i < nseq; i++) id[i] = i;
    return set_slots(c, id.data(), nseq);
}

// Below this many rows the GEMM tiles are mostly padding and the decode kernels are faster.
#define MLH_PREFILL_GEMM_MIN_ROWS 16

static int prefill_token_by_token(mlh_ctx* c, int seq, const int32_t* ids, int n) {
    int rc;
    if ((rc = set_slots(c, &seq, 1))) return rc;
    MLH_CHECK(c, hipMemcpyAsync(c->d_prompt, ids, (size_t)n * 4, hipMemcpyHostToDevice, c->stream));
    for (int i = 0; i < n; i++)
        if ((rc = mlh_launch_step(c, 1, c->d_prompt + i, i == n - 1))) return rc;
    MLH_CHECK(c, hipStreamSynchronize(c->stream));
    c->h_len[seq] += n;
    return 0;
}

extern "C" int mlh_prefill_batch(mlh_ctx* c, int nseg, const int32_t* seqs, const int32_t* ids, const int32_t* lens) {
    int rc = check_ready(c);
    if (rc) return rc;
    const mlh_hparams& hp = c->hp;
    if (nseg <= 0 || nseg > hp.maxSeqs || !seqs || !ids || !lens) { c->err = "bad argument"; return -1; }
    std::vector<char> seen(hp.maxSeqs, 0);
    long total = 0;
    for (int s = 0; s < nseg; s++) {
        if (seqs[s] < 0 || seqs[s] >= hp.maxSeqs || seen[seqs[s]]) { c->err = "sequence indices must be distinct and in range"; return -1; }
        seen[seqs[s]] = 1;
        if (lens[s] <= 0) { c->err = "empty prompt"; return -1; }
        if (c->h_len[seqs[s]] + lens[s] > hp.maxL) { c->err = "prompt does not fit in maxL"; return -1; }
        total += lens[s];
    }
    for (long i = 0; i < total; i++)
        if (ids[i] < 0 || ids[i] >= hp.vocabSize) { c->err = "token id out of range"; return -1; }
    if (c->prefillMode == 0 && total >= MLH_PREFILL_GEMM_MIN_ROWS && mlh_prefill_gemm_supported(c))
        return mlh_run_prefill_gemm(c, nseg, seqs, ids, lens, nullptr);
    long off = 0;
    for (int s = 0; s < nseg; s++) {
        if ((rc = prefill_token_by_token(c, seqs[s], ids + off, lens[s]))) return rc;
        off += lens[s];
    }
    return 0;
}

extern "C" int mlh_prefill(mlh_ctx* c, int seq, const int32_t* ids, int n) {
    return mlh_prefill_batch(c, 1, &seq, ids, &n);
}

// Teacher-forced forward over n tokens appended to `seq`: what runInference(L) leaves in vocabScores_DEVICE and
// vocabScores_postSoftmax_DEVICE for all L columns (inference.cu:723-749), plus the mean next-token cross-entropy.
extern "C" int mlh_forward_full(mlh_ctx* c, int seq, const int32_t* ids, int n, float* logitsOut, float* probsOut, float* meanNll) {
    int rc = check_ready(c);
    if (rc) return rc;
    const mlh_hparams& hp = c->hp;
    const size_t V = hp.vocabSize;
    if (seq < 0 || seq >= hp.maxSeqs) { c->err = "sequence index out of range"; return -1; }
    if (!ids || n <= 0) { c->err = "empty input"; return -1; }
    if (c->h_len[seq] + n > hp.maxL) { c->err = "input does not fit in maxL"; return -1; }
    for (int i = 0; i < n; i++)
        if (ids[i] < 0 || ids[i] >= hp.vocabSize) { c->err = "token id out of range"; return -1; }
    float *dLogits = nullptr, *dProbs = nullptr, *dNll = nullptr;
    int* dTarget = nullptr;
    std::vector<int> target(n, -1);
    for (int i = 0; i + 1 < n; i++) target[i] = ids[i + 1];
    std::vector<float> nll(n, 0.f);
    hipError_t e = hipMalloc((void**)&dLogits, (size_t)n * V * 4);
    if (e == hipSuccess && probsOut) e = hipMalloc((void**)&dProbs, (size_t)n * V * 4);
    if (e == hipSuccess) e = hipMalloc((void**)&dNll, (size_t)n * 4);
    if (e == hipSuccess) e = hipMalloc((void**)&dTarget, (size_t)n * 4);
    if (e == hipSuccess) e = hipMemcpy(dTarget, target.data(), (size_t)n * 4, hipMemcpyHostToDevice);
    if (e != hipSuccess) { c->err = std::string("forward_full buffers: ") + hipGetErrorString(e); rc = -2; }
    if (rc == 0) {
        if (c->prefillMode == 0 && n >= MLH_PREFILL_GEMM_MIN_ROWS && mlh_prefill_gemm_supported(c)) {
            rc = mlh_run_prefill_gemm(c, 1, &seq, ids, &n, dLogits);
        } else { // token by token through the decode kernels, LM head at every position
            rc = set_slots(c, &seq, 1);
            if (rc == 0 && hipMemcpyAsync(c->d_prompt, ids, (size_t)n * 4, hipMemcpyHostToDevice, c->stream) != hipSuccess) rc = -2;
            for (int i = 0; i < n && rc == 0; i++) {
                rc = mlh_launch_step(c, 1, c->d_prompt + i, true);
                if (rc == 0 && hipMemcpyAsync(dLogits + (size_t)i * V, c->logits + (size_t)seq * V, V * 4, hipMemcpyDeviceToDevice, c->stream) != hipSuccess) rc = -2;
            }
            if (rc == 0) { if (hipStreamSynchronize(c->stream) != hipSuccess) rc = -2; else c->h_len[seq] += n; }
            if (rc == -2 && c->err.empty()) c->err = "forward_full: HIP call failed";
        }
    }
    if (rc == 0) rc = mlh_launch_softmax_rows(c, dLogits, dProbs, dTarget, dNll, n);
    if (rc == 0) {
        e = hipStreamSynchronize(c->stream);
        if (e == hipSuccess && logitsOut) e = hipMemcpy(logitsOut, dLogits, (size_t)n * V * 4, hipMemcpyDeviceToHost);
        if (e == hipSuccess && probsOut) e = hipMemcpy(probsOut, dProbs, (size_t)n * V * 4, hipMemcpyDeviceToHost);
        if (e == hipSuccess) e = hipMemcpy(nll.data(), dNll, (size_t)n * 4, hipMemcpyDeviceToHost);
        if (e != hipSuccess) { c->err = std::string("forward_full read-back: ") + hipGetErrorString(e); rc = -2; }
    }
    (void)hipFree(dLogits); (void)hipFree(dProbs); (void)hipFree(dNll); (void)hipFree(dTarget);
    if (rc == 0 && meanNll) {
        double s = 0;
        for (int i = 0; i + 1 < n; i++) s += nll[i];
        *meanNll = n > 1 ? (float)(s / (n - 1)) : 0.f;
    }
    return rc;
}

extern "C" int mlh_set_prefill_mode(mlh_ctx* c, int mode) {
    if (!c) return -1;
    if (mode != 0 && mode != 1) { c->err = "prefill mode must be 0 (auto) or 1 (token by token)"; return -1; }
    if (mode != c->prefillMode)
        for (int g = 0; g < 2; g++) // a captured step follows the mode it was captured under
            if (c->graphExec[g]) { (void)hipGraphExecDestroy(c->graphExec[g]); c->graphExec[g] = nullptr; }
    c->prefillMode = mode;
    return 0;
}

// Captures `k` consecutive decode steps into one executable graph (slot 0: one step, slot 1: graphSteps steps).
static int ensure_graph(mlh_ctx* c, int slot, int nseq, int k) {
    if (c->graphExec[slot] && c->graphNseqOf[slot] == nseq && c->graphStepsOf[slot] == k) return 0;
    if (c->graphExec[slot]) { (void)hipGraphExecDestroy(c->graphExec[slot]); c->graphExec[slot] = nullptr; }
    hipGraph_t g = nullptr;
    MLH_CHECK(c, hipStreamBeginCapture(c->stream, hipStreamCaptureModeThreadLocal));
    int rc = 0;
    for (int i = 0; i < k && rc == 0; i++) rc = mlh_launch_step(c, nseq, c->d_tok, true);
    hipError_t e = hipStreamEndCapture(c->stream, &g);
    if (rc) { if (g) (void)hipGraphDestroy(g); return rc; }
    if (e != hipSuccess) { c->err = std::string("hipStreamEndCapture: ") + hipGetErrorString(e); return -2; }
    e = hipGraphInstantiate(&c->graphExec[slot], g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e != hipSuccess) { c->graphExec[slot] = nullptr; c->err = std::string("hipGraphInstantiate: ") + hipGetErrorString(e); return -2; }
    c->graphNseqOf[slot] = nseq;
    c->graphStepsOf[slot] = k;
    return 0;
}

static bool use_persistent(const mlh_ctx* c, int nseq) {
    // (the single-launch kernels fuse the argmax only: sampling runs through the kernel sequence)
    return nseq == 1 && c->usePersistent && c->temperature <= 0.f && mlh_persistent_supported(c);
}

// After the stream has drained: a single-launch decode that gave up a bounded wait leaves its flag set.  The sequence
// is then put back to where it was before the launch, so the caller can run the same steps again another way:
// position, token and the tag counter are written at a kernel's normal end only; K/V rows of the steps that did run
// are written again with the same values; the XCD-rank kernel keeps gated-delta-net states in LDS until its normal
// end; the barrier kernel stores them at every step, and gets them back from the copy taken before its launch.
static int check_persistent_abort(mlh_ctx* c) {
    if (c->d_timing) mlh_dump_persistent_timing(c);
    unsigned flag = 0;
    MLH_CHECK(c, hipMemcpy(&flag, c->d_sync + 64 * 20, 4, hipMemcpyDeviceToHost));
    if (flag) {
        c->err = flag == 2 ? "XCD-rank decode kernel: the workgroups did not spread evenly over the XCDs"
                           : "persistent decode kernel abandoned a wait (were all workgroups resident?)";
        if (c->usePersistent == 3 && mlh_xcd_supported(c)) { // tags of the abandoned launch must not be met again
            int rc = mlh_xcd_reset(c);
            if (rc) return rc;
        } else {
            int rc = mlh_persistent_restore_states(c);
            if (rc) return rc;
        }
        MLH_CHECK(c, hipStreamSynchronize(c->stream));
        return -3;
    }
    return 0;
}

static int run_steps(mlh_ctx* c, int nseq, int steps) {
    int rc;
    if (use_persistent(c, nseq)) return (c->usePersistent == 3 && mlh_xcd_supported(c)) ? mlh_launch_xcd(c, steps) : mlh_launch_persistent(c, steps);
    if (c->graphSteps >= 1) {
        const int k = c->graphSteps;
        int done = 0;
        if (k > 1 && steps >= k) {
            if ((rc = ensure_graph(c, 1, nseq, k))) return rc;
            for (; done + k <= steps; done += k) MLH_CHECK(c, hipGraphLaunch(c->graphExec[1], c->stream));
        }
        if (done < steps) {
            if ((rc = ensure_graph(c, 0, nseq, 1))) return rc;
            for (; done < steps; done++) MLH_CHECK(c, hipGraphLaunch(c->graphExec[0], c->stream));
        }
    } else {
        for (int i = 0; i < steps; i++)
            if ((rc = mlh_launch_step(c, nseq, c->d_tok, true))) return rc;
    }
    return 0;
}

static int check_decode(mlh_ctx* c, const int32_t* ids, int nseq, int steps) {
    int rc = check_ready(c);
    if (rc) return rc;
    const mlh_hparams& hp = c->hp;
    if (nseq <= 0 || nseq > hp.maxSeqs) { c->err = "nseq out of range"; return -1; }
    if (!ids || steps <= 0) { c->err = "bad argument"; return -1; }
    if (steps > c->outCapacity) { c->err = "more steps than maxL"; return -1; }
    for (int s = 0; s < nseq; s++) {
        if (ids[s] < 0 || ids[s] >= hp.vocabSize) { c->err = "token id out of range"; return -1; }
        if (c->h_len[s] + steps > hp.maxL) { c->err = "sequence would exceed maxL"; return -1; }
    }
    if ((rc = mlh_prepare_batch_step(c, nseq))) return rc;
    return set_identity_slots(c, nseq);
}

// The single-launch kernels need every compute unit for themselves.  When one gives up (another process or stream
// holds units), the call is redone as the kernel sequence and the context stays in that mode: the steps cost more,
// the results are the same.  mlh_get_persistent shows the mode in effect, mlh_persistent_fallbacks how often it happened.
static int fall_back_to_kernel_sequence(mlh_ctx* c) {
    c->persistentFallbacks++;
    c->usePersistent = 0;
    return 0;
}

extern "C" int mlh_decode_loop(mlh_ctx* c, const int32_t* first, int nseq, int steps, int32_t* out) {
    int rc = check_decode(c, first, nseq, steps);
    if (rc) return rc;
    if (!out) { c->err = "null output"; return -1; }
    for (int attempt = 0; attempt < 2; attempt++) {
        const bool single = use_persistent(c, nseq);
        MLH_CHECK(c, hipMemcpyAsync(c->d_tok, first, (size_t)nseq * 4, hipMemcpyHostToDevice, c->stream));
        MLH_CHECK(c, hipMemsetAsync(c->d_stepCounter, 0, 4, c->stream));
        if ((rc = run_steps(c, nseq, steps))) return rc;
        MLH_CHECK(c, hipMemcpyAsync(out, c->d_outIds, (size_t)steps * nseq * 4, hipMemcpyDeviceToHost, c->stream));
        MLH_CHECK(c, hipStreamSynchronize(c->stream));
        if (!single || (rc = check_persistent_abort(c)) == 0) break;
        if (rc != -3) return rc;
        fall_back_to_kernel_sequence(c); // and once more, as a sequence of kernels
    }
    for (int s = 0; s < nseq; s++) c->h_len[s] += steps;
    return 0;
}

extern "C" int mlh_decode_step(mlh_ctx* c, const int32_t* last, int nseq, int32_t* next) {
    return mlh_decode_loop(c, last, nseq, 1, next);
}

extern "C" int mlh_time_decode(mlh_ctx* c, const int32_t* first, int nseq, int steps, double* totalMs) {
    int rc = check_decode(c, first, nseq, steps);
    if (rc) return rc;
    if (!totalMs) { c->err = "null output"; return -1; }
    hipEvent_t e0, e1;
    MLH_CHECK(c, hipEventCreate(&e0));
    MLH_CHECK(c, hipEventCreate(&e1));
    float ms = 0.f;
    for (int attempt = 0; attempt < 2; attempt++) {
        const bool single = use_persistent(c, nseq);
        MLH_CHECK(c, hipMemcpyAsync(c->d_tok, first, (size_t)nseq * 4, hipMemcpyHostToDevice, c->stream));
        MLH_CHECK(c, hipMemsetAsync(c->d_stepCounter, 0, 4, c->stream));
        MLH_CHECK(c, hipStreamSynchronize(c->stream));
        MLH_CHECK(c, hipEventRecord(e0, c->stream));
        rc = run_steps(c, nseq, steps);
        MLH_CHECK(c, hipEventRecord(e1, c->stream));
        MLH_CHECK(c, hipEventSynchronize(e1));
        MLH_CHECK(c, hipEventElapsedTime(&ms, e0, e1));
        if (rc) break;
        if (!single || (rc = check_persistent_abort(c)) == 0) break;
        if (rc != -3) break;
        fall_back_to_kernel_sequence(c);
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc) return rc;
    *totalMs = ms;
    for (int s = 0; s < nseq; s++) c->h_len[s] += steps;
    return 0;
}

extern "C" int mlh_profile_decode(mlh_ctx* c, const int32_t* first, int nseq, int steps, double* usPerLaunch,
                                  int32_t* launchesPerStep) {
    int rc = check_decode(c, first, nseq, steps);
    if (rc) return rc;
    if (!usPerLaunch || !launchesPerStep || steps > 64) { c->err = "bad argument (at most 64 steps)"; return -1; }
    std::vector<hipEvent_t> events;
    std::vector<int> ids;
    hipEvent_t e0;
    MLH_CHECK(c, hipEventCreate(&e0));
    MLH_CHECK(c, hipMemcpyAsync(c->d_tok, first, (size_t)nseq * 4, hipMemcpyHostToDevice, c->stream));
    MLH_CHECK(c, hipMemsetAsync(c->d_stepCounter, 0, 4, c->stream));
    MLH_CHECK(c, hipStreamSynchronize(c->stream));
    c->profEvents = &events;
    c->profIds = &ids;
    std::vector<size_t> stepStart;
    for (int i = 0; i < steps && rc == 0; i++) {
        stepStart.push_back(events.size());
        if (i == 0) { // start marker; later steps measure from the previous step's last kernel
            (void)hipEventRecord(e0, c->stream);
            events.push_back(e0);
            ids.push_back(-1);
        }
        rc = mlh_launch_step(c, nseq, c->d_tok, true);
    }
    c->profEvents = nullptr;
    c->profIds = nullptr;
    hipError_t e = hipStreamSynchronize(c->stream);
    double sum[MLH_K_COUNT] = {0};
    long cnt[MLH_K_COUNT] = {0};
    if (rc == 0 && e == hipSuccess) {
        for (size_t i = 1; i < events.size(); i++) {
            float ms = 0.f;
            if (ids[i] < 0 || hipEventElapsedTime(&ms, events[i - 1], events[i]) != hipSuccess || ms < 0.f) continue;
            sum[ids[i]] += (double)ms * 1000.0;
            cnt[ids[i]]++;
        }
    }
    for (size_t i = 1; i < events.size(); i++) (void)hipEventDestroy(events[i]);
    (void)hipEventDestroy(e0);
    if (rc) return rc;
    if (e != hipSuccess) { c->err = std::string("hipStreamSynchronize: ") + hipGetErrorString(e); return -2; }
    for (int k = 0; k < MLH_K_COUNT; k++) {
        usPerLaunch[k] = cnt[k] ? sum[k] / (double)cnt[k] : 0.0;
        launchesPerStep[k] = (int32_t)(cnt[k] / steps);
    }
    for (int s = 0; s < nseq; s++) c->h_len[s] += steps;
    return 0;
}

extern "C" int mlh_read_logits(mlh_ctx* c, int seq, float* out) {
    int rc = check_ready(c);
    if (rc) return rc;
    if (seq < 0 || seq >= c->hp.maxSeqs || !out) { c->err = "bad argument"; return -1; }
    MLH_CHECK(c, hipStreamSynchronize(c->stream));
    MLH_CHECK(c, hipMemcpy(out, c->logits + (size_t)seq * c->hp.vocabSize, (size_t)c->hp.vocabSize * 4, hipMemcpyDeviceToHost));
    return 0;
}

extern "C" int mlh_read_probs(mlh_ctx* c, int seq, float* out) {
    int rc = check_ready(c);
    if (rc) return rc;
    if (seq < 0 || seq >= c->hp.maxSeqs || !out) { c->err = "bad argument"; return -1; }
    if ((rc = mlh_launch_probs(c, seq))) return rc;
    MLH_CHECK(c, hipStreamSynchronize(c->stream));
    MLH_CHECK(c, hipMemcpy(out, c->probs, (size_t)c->hp.vocabSize * 4, hipMemcpyDeviceToHost));
    return 0;
}

extern "C" int mlh_set_sampling(mlh_ctx* c, float temperature, unsigned long long seed) {
    if (!c) return -1;
    if (!(temperature >= 0.f) || temperature > 1.0e4f) { c->err = "sampling temperature must be in [0, 1e4]"; return -1; }
    if (c->temperature != temperature || c->sampleSeed != seed)
        for (int g = 0; g < 2; g++) // recorded launches carry the old values in their kernel arguments
            if (c->graphExec[g]) { (void)hipGraphExecDestroy(c->graphExec[g]); c->graphExec[g] = nullptr; }
    c->temperature = temperature;
    c->sampleSeed = seed;
    return 0;
}

extern "C" int mlh_set_graph(mlh_ctx* c, int stepsPerGraph) {
    if (!c) return -1;
    if (stepsPerGraph < 0 || stepsPerGraph > 64) { c->err = "steps per graph must be 0..64"; return -1; }
    c->graphSteps = stepsPerGraph;
    return 0;
}

extern "C" int mlh_set_persistent(mlh_ctx* c, int enabled) {
    if (!c) return -1;
    if (enabled != 0 && enabled != 1 && enabled != 3) { c->err = "persistent mode must be 0, 1 or 3"; return -1; }
    c->usePersistent = enabled;
    return 0;
}

extern "C" int mlh_get_persistent(mlh_ctx* c) { return c ? c->usePersistent : -1; }
extern "C" int mlh_persistent_fallbacks(mlh_ctx* c) { return c ? c->persistentFallbacks : -1; }

extern "C" int mlh_debug_inject_abort(mlh_ctx* c, int launches) {
    if (!c || launches < 0) return -1;
    c->injectAbort = launches;
    return 0;
}

extern "C" int mlh_debug_inject_abort_at_step(mlh_ctx* c, int step) {
    if (!c || step < 0) return -1;
    c->injectAbortStep = step;
    return 0;
}

extern "C" int mlh_debug_set_xcd_tag(mlh_ctx* c, unsigned tagsUsed) {
    int rc = check_ready(c);
    if (rc) return rc;
    MLH_CHECK(c, hipStreamSynchronize(c->stream));
    MLH_CHECK(c, hipMemcpy(c->d_sync + 64 * 21, &tagsUsed, 4, hipMemcpyHostToDevice));
    c->xcdTagNext = tagsUsed;
    return 0;
}

extern "C" int mlh_xcd_decode_supported(mlh_ctx* c) { return c && mlh_xcd_supported(c) ? 1 : 0; }

extern "C" int mlh_synchronize(mlh_ctx* c) {
    if (!c) return -1;
    (void)hipSetDevice(c->device);
    MLH_CHECK(c, hipStreamSynchronize(c->stream));
    return 0;
}

extern "C" int mlh_time_kernel(mlh_ctx* c, int kernel, int layer, int nseq, int iters, double* avgUs,
                               double* algoBytes) {
    int rc = check_ready(c);
    if (rc) return rc;
    if (kernel < 0 || kernel >= MLH_K_COUNT || layer < 0 || layer >= c->hp.transformers || nseq <= 0 ||
        nseq > c->hp.maxSeqs || iters <= 0 || !avgUs) { c->err = "bad argument"; return -1; }
    if ((rc = set_identity_slots(c, nseq))) return rc;
    for (int s = 0; s < nseq; s++)
        if (c->h_len[s] >= c->hp.maxL) { c->err = "sequence is full"; return -1; }
    hipEvent_t e0, e1;
    MLH_CHECK(c, hipEventCreate(&e0));
    MLH_CHECK(c, hipEventCreate(&e1));
    for (int i = 0; i < 3; i++)
        if ((rc = mlh_launch_one(c, kernel, layer, nseq))) return rc;
    MLH_CHECK(c, hipEventRecord(e0, c->stream));
    for (int i = 0; i < iters; i++)
        if ((rc = mlh_launch_one(c, kernel, layer, nseq))) return rc;
    MLH_CHECK(c, hipEventRecord(e1, c->stream));
    MLH_CHECK(c, hipEventSynchronize(e1));
    float ms = 0.f;
    MLH_CHECK(c, hipEventElapsedTime(&ms, e0, e1));
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    *avgUs = (double)ms * 1000.0 / iters;
    if (algoBytes) *algoBytes = mlh_kernel_bytes(c, kernel, layer, nseq);
    return 0;
}
