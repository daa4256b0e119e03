/* Host build of plow_amd/csrc/pm_expf.h compared with the C library's expf. Test infrastructure.
 * usage: pm_expf_check <stride>   (stride 1 = all 2^32 bit patterns). Prints the mismatch count. */
#include <math.h>
#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "../plow_amd/csrc/pm_expf.h"

typedef struct { uint64_t lo, hi, stride, bad; } Job;
static void* work(void* p) {
    Job* j = p;
    for (uint64_t u = j->lo; u < j->hi; u += j->stride) {
        const uint32_t b = (uint32_t)u;
        float x, a, c;
        memcpy(&x, &b, 4);
        a = pm_expf(x);
        c = expf(x);
        if (memcmp(&a, &c, 4) != 0 && !(a != a && c != c)) j->bad++;
    }
    return NULL;
}
int main(int argc, char** argv) {
    const uint64_t stride = argc > 1 ? strtoull(argv[1], NULL, 10) : 1;
    enum { NT = 8 };
    pthread_t th[NT];
    Job jobs[NT];
    for (int i = 0; i < NT; i++) {
        jobs[i] = (Job){((uint64_t)i << 32) / NT, ((uint64_t)(i + 1) << 32) / NT, stride, 0};
        pthread_create(&th[i], NULL, work, &jobs[i]);
    }
    uint64_t bad = 0;
    for (int i = 0; i < NT; i++) { pthread_join(th[i], NULL); bad += jobs[i].bad; }
    printf("%llu\n", (unsigned long long)bad);
    return bad != 0;
}
