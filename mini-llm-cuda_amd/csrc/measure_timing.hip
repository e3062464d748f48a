// Measurement only: decodes the constant-rate clock stamps that the single-launch decode kernels leave in
// mlh_ctx::d_timing (allocated only when MLH_PERSIST_TIMING is set when the context is created) and prints the mean
// time per phase to stderr.  Nothing on the product path depends on this file's output.
#include <stdio.h>

#include <algorithm>
#include <vector>

#include "mlh_internal.h"

void mlh_dump_persistent_timing(mlh_ctx* c) {
    if (!c->d_timing) return;
    const int n = 16 * c->hp.transformers;
    std::vector<unsigned long long> t(n);
    if (hipMemcpy(t.data(), c->d_timing, (size_t)n * 8, hipMemcpyDeviceToHost) != hipSuccess) return;
    const char* names[15] = {"A.norm", "A.rows", "A->B sync", "B.mix", "B->C sync", "C.prologue", "C.rows", "C->D sync",
                                    "D.norm", "D.rows", "D->E sync", "E.load", "E.rows", "E->A sync", "x.load"};
    double tot[15] = {0};
    const bool xcd = c->usePersistent == 3 && mlh_xcd_supported(c);
    for (int l = 0; l < c->hp.transformers; l++)
        for (int k = 0; k < (xcd ? 5 : 15); k++) tot[k] += (double)(t[l * 16 + k + 1] - t[l * 16 + k]) / 100.0; // 100 MHz clock
    static const char* tnames[15] = {"x.wait", "A.norm", "A.rows", "B.mix", "C.wait", "C.rows", "h1.wait", "D.norm", "D.rows",
                                     "u.wait", "E.rows", "-", "-", "-", "-"};
    static const char* xnames[15] = {"x.exchange", "A+hop", "B+hop", "C+2hops", "D+hop", "-", "-", "-", "-", "-", "-", "-", "-", "-", "-"};
    if (c->usePersistent == 2) for (int k = 0; k < 15; k++) names[k] = tnames[k];
    if (xcd) for (int k = 0; k < 15; k++) names[k] = xnames[k];
    if (xcd) { // skew between workgroups at four points of the last layer pass
        std::vector<unsigned long long> sk(4 * 256);
        if (hipMemcpy(sk.data(), c->d_timing + 16 * (c->hp.transformers + 1), sk.size() * 8, hipMemcpyDeviceToHost) == hipSuccess) {
            {   // per workgroup with a unit on wave 0: wait for the tile, unit, combine
                std::vector<double> a1, a2, a3;
                for (int w = 0; w < 256; w++)
                    if (sk[4 * w] && sk[4 * w + 1]) {
                        a1.push_back(((double)sk[4 * w + 3] - (double)sk[4 * w + 1]) / 100.0);
                        a2.push_back(((double)sk[4 * w] - (double)sk[4 * w + 3]) / 100.0);
                        a3.push_back(((double)sk[4 * w + 2] - (double)sk[4 * w]) / 100.0);
                    }
                auto pr = [&](const char* nm, std::vector<double>& v) { std::sort(v.begin(), v.end()); if (!v.empty()) fprintf(stderr, "[xcd unit] %-28s n %zu min %.2f median %.2f max %.2f us\n", nm, v.size(), v[0], v[v.size() / 2], v.back()); };
                pr("barrier 2 -> tile waited for", a1); pr("tile ready -> unit end", a2); pr("unit end -> combine done", a3);
            }
            const char* what[4] = {"attention wave 0 end", "wave 0 unit start", "wave 0 combine done", "wave 0 tile ready"};
            unsigned long long t0 = ~0ull;
            for (int w = 0; w < 256; w++) if (sk[4 * w]) t0 = std::min(t0, sk[4 * w]);
            for (int k = 0; k < 4; k++) {
                std::vector<double> v;
                for (int w = 0; w < 256; w++) v.push_back(sk[4 * w + k] ? ((double)sk[4 * w + k] - (double)t0) / 100.0 : -1.0);
                double perX[8] = {0};
                std::vector<double> sorted = v;
                std::sort(sorted.begin(), sorted.end());
                const size_t first = std::lower_bound(sorted.begin(), sorted.end(), 0.0) - sorted.begin(), cnt = 256 - first;
                if (!cnt) continue;
                fprintf(stderr, "[xcd skew] %-20s n %zu min %.2f median %.2f max %.2f us (first 8 workgroups:", what[k], cnt, sorted[first], sorted[first + cnt / 2], sorted[255]);
                for (int w = 0; w < 8; w++) fprintf(stderr, " %.2f", v[w]);
                fprintf(stderr, ")\n");
                (void)perX;
            }
        }
    }
    if (xcd) { // raw stamps relative to the start of the layer pass: communicator 0-9, worker wave 0 10-14
        double rel[16] = {0};
        for (int l = 0; l < c->hp.transformers; l++)
            for (int k = 0; k < 16; k++) rel[k] += ((double)t[l * 16 + k] - (double)t[l * 16]) / 100.0 / c->hp.transformers;
        for (int l = 0; l < c->hp.transformers; l++) {
            fprintf(stderr, "[xcd layer %2d]", l);
            for (int k = 0; k < 16; k++) fprintf(stderr, " %d:%.2f", k, t[l * 16 + k] ? ((double)t[l * 16 + k] - (double)t[l * 16]) / 100.0 : -1.0);
            fprintf(stderr, "\n");
        }
        fprintf(stderr, "[xcd stamps, us from layer start] x: partials seen %.2f gathered %.2f | worker A %.2f..%.2f | q,k,v in LDS %.2f | "
                        "wave 0: units done %.2f combine done %.2f | worker C %.2f..%.2f | h1: partials seen %.2f gathered %.2f | worker D end %.2f | "
                        "u in LDS %.2f | worker E end %.2f\n",
                rel[6], rel[1], rel[10], rel[11], rel[2], rel[12], rel[15], rel[13], rel[14], rel[8], rel[4], rel[7], rel[5], rel[9]);

    }
    fprintf(stderr, "[persistent decode, workgroup 0, last step] mean us per layer:");
    double sum = 0;
    for (int k = 0; k < 15; k++) { fprintf(stderr, " %s=%.2f", names[k], tot[k] / c->hp.transformers); sum += tot[k] / c->hp.transformers; }
    fprintf(stderr, " | layer total %.2f\n", sum);
}

