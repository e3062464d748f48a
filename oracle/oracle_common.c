/* Type-independent parts of the CPU oracle (test infrastructure only; see oracle.h). */
#include <math.h>
#include <stdint.h>
#include <string.h>

#include "oracle.h"

/* inference.cu:364-374, statement for statement: theta is the float product of the
 * int position and powf(base, -2.0f*i/headDim); cosf/sinf of that float. */
void orc_rope_table(float* tab, int maxL, int headDim, float base) {
    int numPairs = headDim / 2;
    for (int col = 0; col < maxL; col++) {
        for (int pair = 0; pair < numPairs; pair++) {
            float theta = col * powf(base, (-2.0f * pair / headDim));
            tab[(size_t)col * headDim + pair * 2] = cosf(theta);
            tab[(size_t)col * headDim + pair * 2 + 1] = sinf(theta);
        }
    }
}

/* fp32 -> bf16 (round to nearest, ties to even) -> fp32.  NaN is kept quiet. */
void orc_round_bf16(float* w, long n) {
    for (long i = 0; i < n; i++) {
        uint32_t u;
        memcpy(&u, &w[i], 4);
        if ((u & 0x7fffffffu) > 0x7f800000u) {
            u |= 0x00400000u;
            u &= 0xffff0000u;
        } else {
            u += 0x7fffu + ((u >> 16) & 1u);
            u &= 0xffff0000u;
        }
        memcpy(&w[i], &u, 4);
    }
}
