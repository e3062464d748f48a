/*
 * Body of the CPU oracle, compiled once per arithmetic type.
 * TEST INFRASTRUCTURE ONLY (see oracle.h).  Before including define:
 *   REAL       float | double
 *   FN(name)   name##_f32 | name##_f64
 *   R_EXP R_SQRT R_LOG1P   libm functions of that type
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "oracle.h"

#define ORC_RMS_EPS ((REAL)1e-8f) /* inference.cu:48,79 */
#define ORC_L2_EPS ((REAL)1e-6f)  /* GDN q/k L2 normalisation */

/* y = W x, W row-major [rows, cols] of float.  (cuBLAS call sites
 * inference.cu:401-465,487-507,582-602,624-695,723-743 all reduce to this
 * per column.)  Sequential accumulation order, one accumulator per row. */
void FN(orc_matvec)(const float* W, const REAL* x, int rows, int cols, REAL* y) {
#pragma omp parallel for schedule(static) if ((long)rows * cols > 65536)
    for (int r = 0; r < rows; r++) {
        const float* w = W + (size_t)r * cols;
        REAL acc = 0;
        for (int c = 0; c < cols; c++) acc += (REAL)w[c] * x[c];
        y[r] = acc;
    }
}

/* Y[l] = W X[l] for L vectors at once (X: [L, ldx], Y: [L, ldy], one vector per row).  Every output
 * element is accumulated exactly as orc_matvec does it (one accumulator, columns in ascending order, a
 * multiply and an add per term), so the result is bit-identical to L calls of orc_matvec; only the loop
 * nest differs: ORC_TB vectors are transposed into a block so that a weight row is read once per block
 * and the independent accumulators of the block's vectors fill the SIMD lanes. */
#define ORC_TB 16
__attribute__((target_clones("avx512f", "avx2", "default"), optimize("O3")))
static void FN(orc_mm_tile)(const float* w0, const float* w1, const float* w2, const float* w3, int cols,
                            const REAL* xT, REAL* out) {
    REAL a0[ORC_TB], a1[ORC_TB], a2[ORC_TB], a3[ORC_TB];
    for (int l = 0; l < ORC_TB; l++) a0[l] = a1[l] = a2[l] = a3[l] = 0;
    for (int c = 0; c < cols; c++) {
        const REAL* xc = xT + (size_t)c * ORC_TB;
        REAL v0 = (REAL)w0[c], v1 = (REAL)w1[c], v2 = (REAL)w2[c], v3 = (REAL)w3[c];
        for (int l = 0; l < ORC_TB; l++) {
            a0[l] += v0 * xc[l];
            a1[l] += v1 * xc[l];
            a2[l] += v2 * xc[l];
            a3[l] += v3 * xc[l];
        }
    }
    for (int l = 0; l < ORC_TB; l++) {
        out[l] = a0[l];
        out[ORC_TB + l] = a1[l];
        out[2 * ORC_TB + l] = a2[l];
        out[3 * ORC_TB + l] = a3[l];
    }
}

void FN(orc_matmat)(const float* W, const REAL* X, int ldx, int rows, int cols, int L, REAL* Y, int ldy) {
    REAL* xT = (REAL*)malloc(sizeof(REAL) * (size_t)cols * ORC_TB);
    for (int l0 = 0; l0 < L; l0 += ORC_TB) {
        int nl = L - l0 < ORC_TB ? L - l0 : ORC_TB;
        for (int c = 0; c < cols; c++)
            for (int l = 0; l < ORC_TB; l++)
                xT[(size_t)c * ORC_TB + l] = l < nl ? X[(size_t)(l0 + l) * ldx + c] : (REAL)0;
#pragma omp parallel for schedule(static)
        for (int r0 = 0; r0 < rows; r0 += 4) {
            REAL out[4 * ORC_TB];
            const float* w[4];
            for (int i = 0; i < 4; i++) w[i] = W + (size_t)(r0 + i < rows ? r0 + i : rows - 1) * cols;
            FN(orc_mm_tile)(w[0], w[1], w[2], w[3], cols, xT, out);
            for (int i = 0; i < 4 && r0 + i < rows; i++)
                for (int l = 0; l < nl; l++) Y[(size_t)(l0 + l) * ldy + r0 + i] = out[i * ORC_TB + l];
        }
    }
    free(xT);
}

/* inference.cu:24-50 + 83-95: r = sqrt(mean(x^2) + eps); y = gamma * (x / r).
 * Division first, then the gain, as the reference's two kernels do. */
void FN(orc_rmsnorm)(const REAL* x, const float* gamma, int n, REAL* y) {
    REAL s = 0;
    for (int i = 0; i < n; i++) s += x[i] * x[i];
    REAL r = R_SQRT(s / (REAL)n + ORC_RMS_EPS);
    for (int i = 0; i < n; i++) y[i] = (REAL)gamma[i] * (x[i] / r);
}

/* inference.cu:52-81 + 97-111: per head RMS over its headDim slice, gamma is
 * indexed by the row inside dim (distinct per head and channel).  In place. */
void FN(orc_head_rmsnorm)(REAL* q, const float* gamma, int heads, int hd) {
    for (int h = 0; h < heads; h++) {
        REAL s = 0;
        for (int i = 0; i < hd; i++) s += q[h * hd + i] * q[h * hd + i];
        REAL r = R_SQRT(s / (REAL)hd + ORC_RMS_EPS);
        for (int i = 0; i < hd; i++) q[h * hd + i] = (REAL)gamma[h * hd + i] * (q[h * hd + i] / r);
    }
}

/* inference.cu:113-134: adjacent pairs (2i, 2i+1) inside each head,
 * cos = tab[pos*hd + 2i], sin = tab[pos*hd + 2i + 1].  In place. */
void FN(orc_rope)(REAL* q, const float* tab, int pos, int heads, int hd) {
    for (int h = 0; h < heads; h++) {
        for (int i = 0; i < hd; i += 2) {
            REAL c = (REAL)tab[(size_t)pos * hd + i];
            REAL s = (REAL)tab[(size_t)pos * hd + i + 1];
            REAL a = q[h * hd + i], b = q[h * hd + i + 1];
            q[h * hd + i] = c * a - s * b;
            q[h * hd + i + 1] = s * a + c * b;
        }
    }
}

/* Causal softmax attention of one query against T cached keys/values
 * (K, V: [T, dim], position-major).  Restates, for the last column only,
 * inference.cu:511-573 with 136-239: s_j = k_j.q / sqrt(hd); m = max (init
 * -1e20); e_j = exp(s_j - m); p_j = e_j / sum e; out = sum p_j v_j. */
void FN(orc_attend)(const REAL* q, const REAL* K, const REAL* V, int T, int dim, int heads, int hd,
                    REAL* out) {
    REAL* s = (REAL*)malloc(sizeof(REAL) * (size_t)T);
    REAL scale = R_SQRT((REAL)hd);
    for (int h = 0; h < heads; h++) {
        REAL m = (REAL)-1.0e20f;
        for (int j = 0; j < T; j++) {
            REAL acc = 0;
            for (int i = 0; i < hd; i++) acc += K[(size_t)j * dim + h * hd + i] * q[h * hd + i];
            s[j] = acc / scale;
            if (s[j] > m) m = s[j];
        }
        REAL sum = 0;
        for (int j = 0; j < T; j++) {
            s[j] = R_EXP(s[j] - m);
            sum += s[j];
        }
        for (int i = 0; i < hd; i++) out[h * hd + i] = 0;
        for (int j = 0; j < T; j++) {
            REAL p = s[j] / sum;
            for (int i = 0; i < hd; i++) out[h * hd + i] += p * V[(size_t)j * dim + h * hd + i];
        }
    }
    free(s);
}

/* Gated-delta-net recurrent update for one head (no reference counterpart).
 * S is [dv, dk] row-major.  With u = S k (a dv-vector):
 *     S <- alpha * (S - beta * u k^T) + beta * v k^T
 *        = alpha * S * (I - beta k k^T) + beta * v k^T
 *     o  = S q   (with the updated S)
 */
void FN(orc_gdn_step)(REAL* S, const REAL* q, const REAL* k, const REAL* v, REAL alpha, REAL beta,
                      int dk, int dv, REAL* o) {
    for (int r = 0; r < dv; r++) {
        REAL* row = S + (size_t)r * dk;
        REAL u = 0;
        for (int c = 0; c < dk; c++) u += row[c] * k[c];
        REAL acc = 0;
        for (int c = 0; c < dk; c++) {
            row[c] = alpha * (row[c] - beta * u * k[c]) + beta * v[r] * k[c];
            acc += row[c] * q[c];
        }
        o[r] = acc;
    }
}

static REAL FN(orc_silu)(REAL v) { return v / ((REAL)1 + R_EXP(-v)); }    /* inference.cu:262-271 */
static REAL FN(orc_sigmoid)(REAL v) { return (REAL)1 / ((REAL)1 + R_EXP(-v)); } /* inference.cu:248 */
static REAL FN(orc_softplus)(REAL v) {
    return (v > 0 ? v : (REAL)0) + R_LOG1P(R_EXP(v > 0 ? -v : v));
}

static void FN(orc_l2norm_heads)(REAL* q, int heads, int hd) {
    for (int h = 0; h < heads; h++) {
        REAL s = 0;
        for (int i = 0; i < hd; i++) s += q[h * hd + i] * q[h * hd + i];
        REAL r = R_SQRT(s + ORC_L2_EPS);
        for (int i = 0; i < hd; i++) q[h * hd + i] = q[h * hd + i] / r;
    }
}

static int FN(orc_argmax)(const REAL* v, int n) {
    int best = 0; /* lowest index wins ties */
    for (int i = 1; i < n; i++)
        if (v[i] > v[best]) best = i;
    return best;
}

/* ------------------------------------------------------------------------ */
/* Cached decode: one token per call, K/V rows and GDN states kept between    */
/* calls.  Invariant tested in tests/: logits of step t equal the last column */
/* of orc_forward_full on the first t+1 tokens.                               */
/* ------------------------------------------------------------------------ */

typedef struct {
    orc_hparams hp;
    const orc_weights* w;
    float* rope;
    int pos;
    REAL* K[ORC_MAX_LAYERS];
    REAL* V[ORC_MAX_LAYERS];
    REAL* S[ORC_MAX_LAYERS];
    REAL *x, *xn, *q, *k, *v, *g, *a, *h1, *hn, *g1, *g2, *u, *tmp, *ple, *xf;
} FN(orc_state);

static int FN(orc_max3)(int a, int b, int c) { return a > b ? (a > c ? a : c) : (b > c ? b : c); }

void* FN(orc_state_new)(const orc_hparams* hp, const orc_weights* w) {
    FN(orc_state)* st = (FN(orc_state)*)calloc(1, sizeof(*st));
    st->hp = *hp;
    st->w = w;
    st->rope = (float*)malloc(sizeof(float) * (size_t)hp->maxL * hp->headDim);
    orc_rope_table(st->rope, hp->maxL, hp->headDim, hp->ropeDenomBase);
    int qd = FN(orc_max3)(hp->dim, hp->gdnHeads * hp->gdnDk, hp->gdnHeads * hp->gdnDv);
    for (int t = 0; t < hp->transformers; t++) {
        if (hp->layerKinds[t] == ORC_KIND_GDN) {
            st->S[t] = (REAL*)calloc((size_t)hp->gdnHeads * hp->gdnDk * hp->gdnDv, sizeof(REAL));
        } else {
            st->K[t] = (REAL*)calloc((size_t)hp->maxL * hp->dim, sizeof(REAL));
            st->V[t] = (REAL*)calloc((size_t)hp->maxL * hp->dim, sizeof(REAL));
        }
    }
#define ORC_ALLOC(f, n) st->f = (REAL*)calloc((size_t)(n), sizeof(REAL))
    ORC_ALLOC(x, hp->dim); ORC_ALLOC(xn, hp->dim); ORC_ALLOC(q, qd); ORC_ALLOC(k, qd);
    ORC_ALLOC(v, qd); ORC_ALLOC(g, qd); ORC_ALLOC(a, qd); ORC_ALLOC(h1, hp->dim);
    ORC_ALLOC(hn, hp->dim); ORC_ALLOC(g1, hp->ffnDim); ORC_ALLOC(g2, hp->ffnDim);
    ORC_ALLOC(u, hp->ffnDim); ORC_ALLOC(tmp, hp->dim); ORC_ALLOC(ple, hp->pleDim + 1);
    ORC_ALLOC(xf, hp->dim);
#undef ORC_ALLOC
    return st;
}

void FN(orc_state_reset)(void* p) {
    FN(orc_state)* st = (FN(orc_state)*)p;
    st->pos = 0;
    for (int t = 0; t < st->hp.transformers; t++)
        if (st->S[t])
            memset(st->S[t], 0, sizeof(REAL) * (size_t)st->hp.gdnHeads * st->hp.gdnDk * st->hp.gdnDv);
}

int FN(orc_state_pos)(void* p) { return ((FN(orc_state)*)p)->pos; }

void FN(orc_state_free)(void* p) {
    FN(orc_state)* st = (FN(orc_state)*)p;
    for (int t = 0; t < ORC_MAX_LAYERS; t++) { free(st->K[t]); free(st->V[t]); free(st->S[t]); }
    free(st->rope); free(st->x); free(st->xn); free(st->q); free(st->k); free(st->v); free(st->g);
    free(st->a); free(st->h1); free(st->hn); free(st->g1); free(st->g2); free(st->u); free(st->tmp);
    free(st->ple); free(st->xf);
    free(st);
}

/* Token mixing of a GDN layer for one position (no reference counterpart):
 *   q,k,v = Wq xn, Wk xn, Wv xn ; q_h,k_h L2-normalised per head ;
 *   alpha_h = exp(-softplus(wa_h.xn + ba_h)) ; beta_h = sigmoid(wb_h.xn + bb_h) ;
 *   state update and read-out as orc_gdn_step.  No RoPE, no QK RMSNorm, no query gating. */
static void FN(orc_gdn_recur)(const orc_hparams* hp, const orc_layer* lw, const REAL* xn, REAL* S,
                              REAL* q, REAL* k, const REAL* v, REAL* a) {
    int Hg = hp->gdnHeads, dk = hp->gdnDk, dv = hp->gdnDv, d = hp->dim;
    FN(orc_l2norm_heads)(q, Hg, dk);
    FN(orc_l2norm_heads)(k, Hg, dk);
#pragma omp parallel for schedule(static) if ((long)Hg * dk * dv > 65536)
    for (int h = 0; h < Hg; h++) {
        REAL za, zb;
        FN(orc_matvec)(lw->gdnWa + (size_t)h * d, xn, 1, d, &za);
        FN(orc_matvec)(lw->gdnWb + (size_t)h * d, xn, 1, d, &zb);
        REAL alpha = R_EXP(-FN(orc_softplus)(za + (REAL)lw->gdnBa[h]));
        REAL beta = FN(orc_sigmoid)(zb + (REAL)lw->gdnBb[h]);
        FN(orc_gdn_step)(S + (size_t)h * dv * dk, q + h * dk, k + h * dk, v + h * dv, alpha, beta, dk,
                         dv, a + h * dv);
    }
}

static void FN(orc_gdn_mix)(const orc_hparams* hp, const orc_layer* lw, const REAL* xn, REAL* S,
                            REAL* q, REAL* k, REAL* v, REAL* a) {
    int Hg = hp->gdnHeads, dk = hp->gdnDk, dv = hp->gdnDv, d = hp->dim;
    FN(orc_matvec)(lw->Wq, xn, Hg * dk, d, q);
    FN(orc_matvec)(lw->Wk, xn, Hg * dk, d, k);
    FN(orc_matvec)(lw->Wv, xn, Hg * dv, d, v);
    FN(orc_gdn_recur)(hp, lw, xn, S, q, k, v, a);
}

/* Per-layer-embedding branch for one position (no reference counterpart):
 *   e = silu(Wpg xn) (*) P[tok]   (pleDim values);   returns Wpu e  in out[dim].
 * It reads the same RMS1-normed input as Q/K/V and is added into the residual
 * together with the output projection:  h1 = Wo a + x + Wpu e. */
static void FN(orc_ple_branch)(const orc_hparams* hp, const orc_layer* lw, const REAL* xn, int token,
                               REAL* e, REAL* out) {
    int p = hp->pleDim, d = hp->dim;
    FN(orc_matvec)(lw->pleGate, xn, p, d, e);
    for (int j = 0; j < p; j++) e[j] = FN(orc_silu)(e[j]) * (REAL)lw->pleTable[(size_t)token * p + j];
    FN(orc_matvec)(lw->pleUp, e, d, p, out);
}

int FN(orc_decode_step)(void* p, int token, REAL* logits) {
    FN(orc_state)* st = (FN(orc_state)*)p;
    const orc_hparams* hp = &st->hp;
    const orc_weights* w = st->w;
    int d = hp->dim, H = hp->attnHeads, hd = hp->headDim, F = hp->ffnDim, pos = st->pos;
    if (pos >= hp->maxL || token < 0 || token >= hp->vocabSize) return -1;

    for (int i = 0; i < d; i++) st->x[i] = (REAL)w->E[(size_t)token * d + i]; /* inference.cu:9-22 */

    for (int t = hp->transformers - 1; t >= 0; t--) { /* inference.cu:384-385 */
        const orc_layer* lw = &w->layers[t];
        int ad; /* width of the mixing output fed to Wo */
        FN(orc_rmsnorm)(st->x, lw->rms1, d, st->xn);
        if (hp->layerKinds[t] == ORC_KIND_GDN) {
            FN(orc_gdn_mix)(hp, lw, st->xn, st->S[t], st->q, st->k, st->v, st->a);
            ad = hp->gdnHeads * hp->gdnDv;
        } else {
            FN(orc_matvec)(lw->Wq, st->xn, d, d, st->q);
            FN(orc_matvec)(lw->Wk, st->xn, d, d, st->k);
            FN(orc_matvec)(lw->Wv, st->xn, d, d, st->v);
            if (hp->qkRmsNorm) { /* inference.cu:467-474, before RoPE */
                FN(orc_head_rmsnorm)(st->q, lw->qRms, H, hd);
                FN(orc_head_rmsnorm)(st->k, lw->kRms, H, hd);
            }
            FN(orc_rope)(st->q, st->rope, pos, H, hd);
            FN(orc_rope)(st->k, st->rope, pos, H, hd);
            memcpy(st->K[t] + (size_t)pos * d, st->k, sizeof(REAL) * d);
            memcpy(st->V[t] + (size_t)pos * d, st->v, sizeof(REAL) * d);
            FN(orc_attend)(st->q, st->K[t], st->V[t], pos + 1, d, H, hd, st->a);
            if (hp->queryGating) { /* inference.cu:486-508, 241-250 */
                FN(orc_matvec)(lw->Wg, st->xn, d, d, st->g);
                for (int i = 0; i < d; i++) st->a[i] = st->a[i] * FN(orc_sigmoid)(st->g[i]);
            }
            ad = d;
        }
        FN(orc_matvec)(lw->Wo, st->a, d, ad, st->h1); /* inference.cu:582-610 */
        for (int i = 0; i < d; i++) st->h1[i] = st->h1[i] + st->x[i];
        if (hp->pleDim > 0) {
            FN(orc_ple_branch)(hp, lw, st->xn, token, st->ple, st->tmp);
            for (int i = 0; i < d; i++) st->h1[i] += st->tmp[i];
        }
        FN(orc_rmsnorm)(st->h1, lw->rms2, d, st->hn); /* inference.cu:612-621 */
        FN(orc_matvec)(lw->W1A, st->hn, F, d, st->g1); /* inference.cu:624-667 */
        FN(orc_matvec)(lw->W1B, st->hn, F, d, st->g2);
        for (int i = 0; i < F; i++) st->u[i] = FN(orc_silu)(st->g1[i]) * st->g2[i]; /* :262-281 */
        FN(orc_matvec)(lw->W2, st->u, d, F, st->tmp); /* inference.cu:675-699 */
        for (int i = 0; i < d; i++) st->x[i] = st->tmp[i] + st->h1[i];
    }
    st->pos = pos + 1;

    FN(orc_rmsnorm)(st->x, w->gammaF, d, st->xf); /* inference.cu:705-715 */
    REAL* out = logits ? logits : (REAL*)malloc(sizeof(REAL) * (size_t)hp->vocabSize);
    FN(orc_matvec)(w->E, st->xf, hp->vocabSize, d, out); /* inference.cu:723-743, tied embedding */
    int best = FN(orc_argmax)(out, hp->vocabSize);
    if (!logits) free(out);
    return best;
}

/* ------------------------------------------------------------------------ */
/* Reference-style full recompute (inference.cu:376-751): every op over all L */
/* columns, explicit [heads, L, L] score matrices, no cache.  Activations are */
/* column-major [feature, position] like the reference: x[pos*dim + row].     */
/* logits/probs: [vocab x L] column-major or NULL ([vocab], last position     */
/* only, when lastOnly != 0); finalHidden: [dim x L] or NULL.                 */
/* ------------------------------------------------------------------------ */
int FN(orc_forward_full)(const orc_hparams* hp, const orc_weights* w, const int* tokens, int L,
                         REAL* logits, REAL* probs, REAL* finalHidden, int lastOnly) {
    int d = hp->dim, H = hp->attnHeads, hd = hp->headDim, F = hp->ffnDim, V = hp->vocabSize;
    if (L <= 0 || L > hp->maxL) return -1;
    int qd = FN(orc_max3)(d, hp->gdnHeads * hp->gdnDk, hp->gdnHeads * hp->gdnDv);
    float* rope = (float*)malloc(sizeof(float) * (size_t)hp->maxL * hd);
    orc_rope_table(rope, hp->maxL, hd, hp->ropeDenomBase);
#define ORC_BUF(name, n) REAL* name = (REAL*)calloc((size_t)(n), sizeof(REAL))
    ORC_BUF(x, (size_t)d * L); ORC_BUF(xn, (size_t)d * L); ORC_BUF(Q, (size_t)qd * L);
    ORC_BUF(K, (size_t)qd * L); ORC_BUF(Vv, (size_t)qd * L); ORC_BUF(G, (size_t)qd * L);
    ORC_BUF(A, (size_t)qd * L); ORC_BUF(h1, (size_t)d * L); ORC_BUF(hn, (size_t)d * L);
    ORC_BUF(g1, (size_t)F * L); ORC_BUF(g2, (size_t)F * L); ORC_BUF(u, (size_t)F * L);
    ORC_BUF(tmp, d); ORC_BUF(ple, hp->pleDim + 1);
    ORC_BUF(Sc, (size_t)H * L * L); /* attnKtQByHead..postSoftmax, network_globals.h:38-43 */
    ORC_BUF(St, (size_t)hp->gdnHeads * hp->gdnDk * hp->gdnDv + 1);
#undef ORC_BUF

    for (int l = 0; l < L; l++) {
        if (tokens[l] < 0 || tokens[l] >= V) return -2;
        for (int r = 0; r < d; r++) x[(size_t)l * d + r] = (REAL)w->E[(size_t)tokens[l] * d + r];
    }

    for (int t = hp->transformers - 1; t >= 0; t--) {
        const orc_layer* lw = &w->layers[t];
        int ad;
        for (int l = 0; l < L; l++) FN(orc_rmsnorm)(x + (size_t)l * d, lw->rms1, d, xn + (size_t)l * d);
        if (hp->layerKinds[t] == ORC_KIND_GDN) {
            int Hg = hp->gdnHeads, dk = hp->gdnDk, dv = hp->gdnDv;
            ad = Hg * dv;
            memset(St, 0, sizeof(REAL) * (size_t)Hg * dk * dv);
            FN(orc_matmat)(lw->Wq, xn, d, Hg * dk, d, L, Q, qd);
            FN(orc_matmat)(lw->Wk, xn, d, Hg * dk, d, L, K, qd);
            FN(orc_matmat)(lw->Wv, xn, d, Hg * dv, d, L, Vv, qd);
            for (int l = 0; l < L; l++) /* recurrence from the zero state, position by position */
                FN(orc_gdn_recur)(hp, lw, xn + (size_t)l * d, St, Q + (size_t)l * qd, K + (size_t)l * qd,
                                  Vv + (size_t)l * qd, A + (size_t)l * ad);
        } else {
            ad = d;
            FN(orc_matmat)(lw->Wq, xn, d, d, d, L, Q, d);
            FN(orc_matmat)(lw->Wk, xn, d, d, d, L, K, d);
            FN(orc_matmat)(lw->Wv, xn, d, d, d, L, Vv, d);
            if (hp->queryGating) FN(orc_matmat)(lw->Wg, xn, d, d, d, L, G, d);
            for (int l = 0; l < L; l++) {
                if (hp->qkRmsNorm) {
                    FN(orc_head_rmsnorm)(Q + (size_t)l * d, lw->qRms, H, hd);
                    FN(orc_head_rmsnorm)(K + (size_t)l * d, lw->kRms, H, hd);
                }
                FN(orc_rope)(Q + (size_t)l * d, rope, l, H, hd);
                FN(orc_rope)(K + (size_t)l * d, rope, l, H, hd);
            }
            /* KtQ per head, S[h][qcol][krow] at h*L*L + qcol*L + krow (inference.cu:511-535),
             * then scale+mask (136-155), column max (157-186), exp+sum (188-218), normalise (220-239). */
            REAL scale = R_SQRT((REAL)hd);
#pragma omp parallel for collapse(2) schedule(dynamic, 8) if (L >= 64)
            for (int h = 0; h < H; h++) {
                for (int qc = 0; qc < L; qc++) {
                    REAL* col = Sc + ((size_t)h * L + qc) * L;
                    for (int kr = 0; kr < L; kr++) {
                        REAL acc = 0;
                        for (int i = 0; i < hd; i++)
                            acc += K[(size_t)kr * d + h * hd + i] * Q[(size_t)qc * d + h * hd + i];
                        col[kr] = (kr > qc) ? (REAL)0 : acc / scale;
                    }
                    REAL m = (REAL)-1.0e20f;
                    for (int kr = 0; kr <= qc; kr++)
                        if (col[kr] > m) m = col[kr];
                    REAL sum = 0;
                    for (int kr = 0; kr <= qc; kr++) {
                        col[kr] = R_EXP(col[kr] - m);
                        sum += col[kr];
                    }
                    for (int kr = 0; kr < L; kr++) col[kr] = (kr <= qc) ? col[kr] / sum : (REAL)0;
                    /* V.P (inference.cu:549-573): all L keys enter the product, masked ones with p = 0 */
                    for (int i = 0; i < hd; i++) {
                        REAL acc = 0;
                        for (int kr = 0; kr < L; kr++) acc += Vv[(size_t)kr * d + h * hd + i] * col[kr];
                        A[(size_t)qc * d + h * hd + i] = acc;
                    }
                }
            }
            if (hp->queryGating)
                for (size_t i = 0; i < (size_t)d * L; i++) A[i] = A[i] * FN(orc_sigmoid)(G[i]);
        }
        FN(orc_matmat)(lw->Wo, A, ad, d, ad, L, h1, d);
        for (int l = 0; l < L; l++) {
            for (int r = 0; r < d; r++) h1[(size_t)l * d + r] += x[(size_t)l * d + r];
            if (hp->pleDim > 0) {
                FN(orc_ple_branch)(hp, lw, xn + (size_t)l * d, tokens[l], ple, tmp);
                for (int r = 0; r < d; r++) h1[(size_t)l * d + r] += tmp[r];
            }
            FN(orc_rmsnorm)(h1 + (size_t)l * d, lw->rms2, d, hn + (size_t)l * d);
        }
        FN(orc_matmat)(lw->W1A, hn, d, F, d, L, g1, F);
        FN(orc_matmat)(lw->W1B, hn, d, F, d, L, g2, F);
        for (size_t i = 0; i < (size_t)F * L; i++) u[i] = FN(orc_silu)(g1[i]) * g2[i];
        FN(orc_matmat)(lw->W2, u, F, d, F, L, x, d); /* x is free from here on: h1 holds the residual */
        for (size_t i = 0; i < (size_t)d * L; i++) x[i] = x[i] + h1[i];
    }

    if (finalHidden) memcpy(finalHidden, x, sizeof(REAL) * (size_t)d * L);
    if (logits || probs) {
        REAL* lg = (REAL*)malloc(sizeof(REAL) * (size_t)V);
        REAL* all = NULL;
        if (!lastOnly) { /* every position: one blocked product over the final-normed columns */
            all = (REAL*)malloc(sizeof(REAL) * (size_t)V * L);
            for (int l = 0; l < L; l++) FN(orc_rmsnorm)(x + (size_t)l * d, w->gammaF, d, xn + (size_t)l * d);
            FN(orc_matmat)(w->E, xn, d, V, d, L, all, V);
        }
        for (int l = lastOnly ? L - 1 : 0; l < L; l++) {
            size_t o = lastOnly ? 0 : (size_t)l * V;
            if (all) {
                memcpy(lg, all + (size_t)l * V, sizeof(REAL) * (size_t)V);
            } else {
                FN(orc_rmsnorm)(x + (size_t)l * d, w->gammaF, d, tmp);
                FN(orc_matvec)(w->E, tmp, V, d, lg);
            }
            if (logits) memcpy(logits + o, lg, sizeof(REAL) * (size_t)V);
            if (probs) { /* inference.cu:293-362 */
                REAL m = (REAL)-1.0e20f, sum = 0;
                for (int i = 0; i < V; i++)
                    if (lg[i] > m) m = lg[i];
                for (int i = 0; i < V; i++) {
                    probs[o + i] = R_EXP(lg[i] - m);
                    sum += probs[o + i];
                }
                for (int i = 0; i < V; i++) probs[o + i] /= sum;
            }
        }
        free(lg);
        free(all);
    }
    free(rope); free(x); free(xn); free(Q); free(K); free(Vv); free(G); free(A); free(h1); free(hn);
    free(g1); free(g2); free(u); free(tmp); free(ple); free(Sc); free(St);
    return 0;
}
