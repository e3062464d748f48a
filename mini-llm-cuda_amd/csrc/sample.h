// Temperature sampling of the next token from a row of logits, fused into the kernels that otherwise take the
// argmax.  The reference has no sampling (its loop keeps the top entry of a qsort, inference_orchestrator.cu:120-165);
// the rule here is the plain one: p_i = exp((l_i - max l) / T) / Z, and the pick is the smallest index i whose
// cumulative sum exceeds u Z, with u a 53-bit uniform in [0, 1) drawn from a counter-based generator keyed by
// (seed, sequence id, position of the token being drawn) -- so a sequence draws the same numbers alone or in a batch,
// eagerly or from a graph.  Sums run in index order in double precision.
#pragma once
#include <stdint.h>

__host__ __device__ inline uint64_t mlh_splitmix64(uint64_t x) { // Steele, Lea, Flood: SplitMix64 output function
    x += 0x9E3779B97F4A7C15ull;
    uint64_t z = x;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
__host__ __device__ inline double mlh_sample_uniform(uint64_t seed, int seq, int pos) {
    const uint64_t base = mlh_splitmix64(mlh_splitmix64(seed) ^ ((uint64_t)(seq + 1) * 0xD1342543DE82EF95ull));
    return (double)(mlh_splitmix64(base + (uint64_t)pos) >> 11) * (1.0 / 9007199254740992.0);
}

// Block-wide draw (NT threads, all must call it): thread t owns the contiguous indices [t seg, (t + 1) seg).
// sd: NT + 1 doubles of LDS, si: one int of LDS.  Returns the picked index in every thread.
template <int NT>
__device__ inline int mlh_sample_row(const float* __restrict__ row, int V, float T, double u, double* sd, int* si) {
    const int tid = threadIdx.x;
    const int seg = (V + NT - 1) / NT, i0 = min(V, tid * seg), i1 = min(V, i0 + seg);
    float mx = -3.0e38f;
    for (int i = i0; i < i1; i++) mx = fmaxf(mx, row[i]);
    sd[tid] = (double)mx;
    __syncthreads();
    if (tid == 0) {
        double m = sd[0];
        for (int t = 1; t < NT; t++) m = fmax(m, sd[t]);
        sd[NT] = m;
    }
    __syncthreads();
    const double m = sd[NT], invT = 1.0 / (double)T;
    __syncthreads();
    double s = 0.0;
    for (int i = i0; i < i1; i++) s += exp(((double)row[i] - m) * invT);
    sd[tid] = s;
    __syncthreads();
    if (tid == 0) { // exclusive prefix over the threads, total in sd[NT]
        double run = 0.0;
        for (int t = 0; t < NT; t++) { const double v = sd[t]; sd[t] = run; run += v; }
        sd[NT] = run;
        *si = V - 1; // stays if rounding leaves the target at or beyond the total
    }
    __syncthreads();
    const double target = u * sd[NT], excl = sd[tid], next = sd[tid + 1];
    if (i0 < i1 && target >= excl && target < next) {
        double part = 0.0;
        int pick = i1 - 1;
        for (int i = i0; i < i1; i++) {
            part += exp(((double)row[i] - m) * invT);
            if (excl + part > target) { pick = i; break; }
        }
        *si = pick;
    }
    __syncthreads();
    return *si;
}
