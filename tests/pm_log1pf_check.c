/* Host build of plow_amd/csrc/pm_log1pf.h compared with the C library's log1pf on every float in [0, 1].
 * Test infrastructure. usage: pm_log1pf_check <stride>   (stride 1 = all bit patterns 0 .. 0x3f800000).
 * Prints the mismatch count. */
#include <math.h>
#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "../plow_amd/csrc/pm_log1pf.h"

typedef struct { uint64_t lo, hi, stride, bad; uint32_t first; } Job;
static void* work(void* p) {
    Job* j = p;
    for (uint64_t u = j->lo; u < j->hi; u += j->stride) {
        const uint32_t b = (uint32_t)u;
        float x, a, c;
        memcpy(&x, &b, 4);
        a = pm_log1pf_unit(x);
        c = log1pf(x);
        if (memcmp(&a, &c, 4) != 0) { if (!j->bad) j->first = b; j->bad++; }
    }
    return NULL;
}
int main(int argc, char** argv) {
    const uint64_t stride = argc > 1 ? strtoull(argv[1], NULL, 10) : 1;
    enum { NT = 8 };
    const uint64_t top = 0x3f800000ull + 1ull;
    pthread_t th[NT];
    Job jobs[NT];
    for (int i = 0; i < NT; i++) {
        jobs[i] = (Job){top * i / NT, top * (i + 1) / NT, stride, 0, 0};
        pthread_create(&th[i], NULL, work, &jobs[i]);
    }
    uint64_t bad = 0;
    for (int i = 0; i < NT; i++) {
        pthread_join(th[i], NULL);
        if (jobs[i].bad && !bad) fprintf(stderr, "first mismatch at bits 0x%08x\n", jobs[i].first);
        bad += jobs[i].bad;
    }
    printf("%llu\n", (unsigned long long)bad);
    return bad != 0;
}
