/* Check of the three-operation division by a level count used by the quantise kernels
 * (veloxquant_mlx_amd/csrc/kivi_quant.hip, group_scale with LevelDiv):
 *     r = RN(1 / L);  q0 = x * r;  e = fma(-q0, L, x);  q = fma(e, r, q0)
 * against x / L in IEEE float32, for L = 2^b - 1, b = 1 .. 8.
 *
 *   exact_level_division <stride>    every stride-th non-negative finite float (the test suite: 4099)
 *   exact_level_division 1           all 2 139 095 040 of them per level count (minutes on 8 cores);
 *                                    last run in full: no mismatch for any of the eight level counts
 *
 * Prints one line per level count and exits with 1 on any mismatch.  Build without FMA contraction
 * (-ffp-contract=off): the products and sums above are the operations being checked. */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

enum { THREADS = 8 };
static const float LEVELS[8] = {1, 3, 7, 15, 31, 63, 127, 255};
typedef struct { float L; uint32_t lo, hi, stride; uint64_t bad; uint32_t first; } job_t;

static void *run(void *p) {
    job_t *j = (job_t *)p;
    const float L = j->L, r = 1.0f / L;
    j->bad = 0;
    for (uint64_t b = j->lo; b < j->hi; b += j->stride) {
        const uint32_t bits = (uint32_t)b;
        float x;
        memcpy(&x, &bits, 4);
        volatile float q0 = x * r;
        volatile float e = fmaf(-q0, L, x);
        volatile float q = fmaf(e, r, q0);
        if (q != x / L) {
            if (!j->bad) j->first = bits;
            ++j->bad;
        }
    }
    return 0;
}

int main(int argc, char **argv) {
    const uint32_t stride = argc > 1 ? (uint32_t)strtoul(argv[1], 0, 10) : 4099u;
    const uint32_t total = 0x7f800000u;   /* bit patterns of the finite non-negative floats */
    int failed = 0;
    if (stride == 0) return 2;
    for (int li = 0; li < 8; ++li) {
        pthread_t th[THREADS];
        job_t jobs[THREADS];
        uint64_t bad = 0;
        uint32_t first = 0;
        for (int t = 0; t < THREADS; ++t) {
            jobs[t].L = LEVELS[li];
            jobs[t].stride = stride;
            jobs[t].lo = (uint32_t)((uint64_t)total * t / THREADS);
            jobs[t].hi = (uint32_t)((uint64_t)total * (t + 1) / THREADS);
            pthread_create(&th[t], 0, run, &jobs[t]);
        }
        for (int t = 0; t < THREADS; ++t) {
            pthread_join(th[t], 0);
            if (jobs[t].bad && !bad) first = jobs[t].first;
            bad += jobs[t].bad;
        }
        printf("levels %g: %llu mismatches", LEVELS[li], (unsigned long long)bad);
        if (bad) printf(" (first at bits 0x%08x)", first);
        printf("\n");
        failed |= bad != 0;
    }
    return failed;
}
