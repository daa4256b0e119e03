/* CPU model of the decode pair kernel's item walk (plow_amd/csrc/plowrt_dec_obj.hip) over the counter
 * protocol of plow_amd/csrc/dec_pair_protocol.h, whose functions it calls: workgroups walk their GLU or
 * DOWN items in order, every access to the counter scratch is one step, and a seeded scheduler
 * interleaves the workgroups' steps at random, sometimes starving the GLU side so that DOWN items give up
 * their bounded wait. Checked over many schedules and two launches in a row on the same scratch:
 *   - a DOWN item only multiplies after every GLU item of its expert has finished; one that gave up
 *     poisons instead;
 *   - no item touches an expert's words after they were reset;
 *   - the scratch is all zero when the launch ends (so the next launch starts clean).
 * `--old-reset` models the earlier rule (the expert's last DOWN item resets the words, a DOWN item that
 * gave up counts like any other) and must FAIL these checks: it shows that the model sees the defect.
 * Exit status: 0 = all checks held, 1 = a check failed. */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../plow_amd/csrc/dec_pair_protocol.h"

#define MAX_E 12
#define MAX_ITEMS 512

static unsigned long long rs = 88172645463325252ull;
static unsigned rnd(void) { rs ^= rs << 13; rs ^= rs >> 7; rs ^= rs << 17; return (unsigned)(rs >> 33); }

typedef struct { int expert, is_down; } Item;
typedef struct {
    int items[MAX_ITEMS], n, cur; /* the workgroup's item list and position */
    int phase;                    /* position inside the current item */
    unsigned polls, before;
    int ready;
} Worker;

enum { P_START, P_WORK, P_ADD_GLU, P_ADD_DONE, P_RESET0, P_RESET2, P_OLD_ADD_DOWN, P_OLD_RESET };

int main(int argc, char** argv) {
    const int old_reset = argc > 1 && !strcmp(argv[1], "--old-reset");
    int failures = 0, gave_up_total = 0;
    for (int trial = 0; trial < 400; trial++) {
        const int E = 1 + (int)(rnd() % MAX_E), G = 1 + (int)(rnd() % 6), D = 1 + (int)(rnd() % 5);
        const int n_glu_w = 1 + (int)(rnd() % 4), n_down_w = 1 + (int)(rnd() % 6);
        const unsigned spin = 1u + rnd() % 6u; /* a tiny limit, so that waits do give up */
        const int starve = (int)(rnd() % 3);   /* how strongly the scheduler prefers DOWN workgroups */
        int live[MAX_E], tile0[MAX_E], tiles = 0;
        for (int e = 0; e < E; e++) { live[e] = rnd() % 5 != 0; tile0[e] = tiles; if (live[e]) tiles += 1 + (int)(rnd() % 3); }
        unsigned* ctr = (unsigned*)calloc((size_t)(tiles + 1) * DP_WORDS_PER_TILE, sizeof(unsigned));
        for (int launch = 0; launch < 2; launch++) {
            Item items[2 * MAX_E * 8];
            int n_items = 0;
            Worker w[16];
            memset(w, 0, sizeof w);
            /* item lists: as the kernel walks them (first, first + stride, ...), skipped experts left out */
            for (int side = 0; side < 2; side++) {
                const int per = side ? D : G, nw = side ? n_down_w : n_glu_w, base = side ? n_glu_w : 0;
                for (int it = 0; it < E * per; it++) {
                    const int e = E - 1 - it / per;
                    if (!live[e]) continue;
                    items[n_items].expert = e, items[n_items].is_down = side;
                    Worker* wk = &w[base + it % nw];
                    wk->items[wk->n++] = n_items++;
                }
            }
            int glu_finished[MAX_E] = {0}, reset_done[MAX_E] = {0};
            const int nw = n_glu_w + n_down_w;
            for (;;) {
                int runnable[16], nr = 0;
                for (int i = 0; i < nw; i++) if (w[i].cur < w[i].n) runnable[nr++] = i;
                if (!nr) break;
                int pick = runnable[rnd() % (unsigned)nr];
                if (starve && pick < n_glu_w && rnd() % (unsigned)(1 + 3 * starve)) { /* try to run a DOWN workgroup instead */
                    for (int i = 0; i < nr; i++) if (runnable[i] >= n_glu_w) { pick = runnable[i + (int)(rnd() % (unsigned)(nr - i))]; break; }
                }
                Worker* wk = &w[pick];
                const Item it = items[wk->items[wk->cur]];
                unsigned* mine = ctr + dp_expert_words((uint32_t)tile0[it.expert]);
#define TOUCH() do { if (reset_done[it.expert]) { printf("trial %d launch %d: expert %d touched after reset\n", trial, launch, it.expert); failures++; } } while (0)
                switch (wk->phase) {
                case P_START:
                    if (!it.is_down) { wk->phase = P_WORK; break; }
                    TOUCH();
                    wk->ready = dp_down_ready(mine[DP_GLU_DONE], (uint32_t)G); /* one poll */
                    if (wk->ready || ++wk->polls >= spin) wk->phase = P_WORK;
                    break;
                case P_WORK:
                    if (it.is_down) {
                        if (wk->ready && glu_finished[it.expert] != G) {
                            printf("trial %d launch %d: DOWN of expert %d ran with %d of %d GLU items done\n", trial, launch, it.expert, glu_finished[it.expert], G);
                            failures++;
                        }
                        if (!wk->ready) gave_up_total++; /* poisons its rows */
                        wk->phase = old_reset ? P_OLD_ADD_DOWN : P_ADD_DONE;
                    } else {
                        glu_finished[it.expert]++;
                        wk->phase = P_ADD_GLU;
                    }
                    break;
                case P_ADD_GLU:
                    TOUCH();
                    mine[DP_GLU_DONE]++;
                    wk->phase = old_reset ? -1 : P_ADD_DONE;
                    break;
                case P_ADD_DONE:
                    TOUCH();
                    wk->before = mine[DP_ITEMS_DONE]++;
                    wk->phase = dp_is_last(wk->before, (uint32_t)G, (uint32_t)D) ? P_RESET0 : -1;
                    break;
                case P_RESET0: mine[DP_GLU_DONE] = 0; wk->phase = P_RESET2; break;
                case P_RESET2: mine[DP_ITEMS_DONE] = 0; reset_done[it.expert] = 1; wk->phase = -1; break;
                case P_OLD_ADD_DOWN: /* the earlier rule: word 1 counts DOWN items, the last one resets */
                    TOUCH();
                    wk->before = mine[1]++;
                    wk->phase = wk->before + 1u == (unsigned)D ? P_OLD_RESET : -1;
                    break;
                case P_OLD_RESET: mine[DP_GLU_DONE] = 0; mine[1] = 0; reset_done[it.expert] = 1; wk->phase = -1; break;
                }
                if (wk->phase == -1) { wk->cur++; wk->phase = P_START; wk->polls = 0; wk->ready = 0; }
            }
            for (int i = 0; i < tiles * (int)DP_WORDS_PER_TILE; i++)
                if (ctr[i]) { printf("trial %d launch %d: scratch word %d left at %u\n", trial, launch, i, ctr[i]); failures++; break; }
            if (failures > 20) break;
        }
        free(ctr);
        if (failures > 20) break;
    }
    printf("dec_pair_model: %d failures, %d waits gave up (%s)\n", failures, gave_up_total, old_reset ? "old reset rule" : "protocol of dec_pair_protocol.h");
    if (!gave_up_total) { printf("no wait gave up: the schedules do not exercise the path\n"); return 1; }
    return failures ? 1 : 0;
}
