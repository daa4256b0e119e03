/* dec_pair_protocol.h — the counter protocol of the decode pair kernel (plowrt_dec_obj.hip), as plain
 * functions so that the kernel and a CPU model of its item walk (tests/dec_pair_model.c) share one
 * statement of it.
 *
 * The caller hands the kernel a zeroed u32 scratch of 4 words per 64-row tile and expects it back zeroed
 * (plow crates/plowrt/src/exec/amd.rs:3416-3430). Expert e owns the four words at 4 * tilep[e] (its first
 * 64-row tile: unique among experts with rows):
 *   word 0  GLU items of the expert that have finished (fq / fs of their 128 channels are visible)
 *   word 2  items of the expert, GLU and DOWN, that have finished
 * A DOWN item polls word 0 until it reaches the expert's GLU item count, at most `spin_limit` times; if it
 * gives up it writes NaN into the part rows it owns (plow's convention for "could not compute",
 * runtime/amd/op_moe.h:5173-5199) instead of multiplying. Every item, whatever happened to it, ends by
 * adding 1 to word 2; the item that brings word 2 to the expert's total zeroes words 0 and 2. Nothing can
 * touch the words after that, because every other item of the expert has already made its last access
 * (its own add to word 2), so the scratch is left zeroed whether or not a wait gave up. Words 1 and 3 are
 * never written.
 *
 * Ordering. The argument above needs an item's add to word 0 to be performed before its add to word 2, and
 * the last item's two reset stores after every other item's accesses; the words are different addresses, so
 * relaxed atomics alone would not order them. The kernel's add to word 2 is therefore an acquire-release
 * operation at device scope (release for every item, acquire for the one that resets). The CPU model walks
 * the items with every access as one sequentially consistent step: it checks the counting, not the memory
 * model. */
#ifndef PLOW_DEC_PAIR_PROTOCOL_H
#define PLOW_DEC_PAIR_PROTOCOL_H

#include <stdint.h>

#ifndef DP_FN
#define DP_FN static inline
#endif

#define DP_WORDS_PER_TILE 4u
#define DP_GLU_DONE 0u
#define DP_ITEMS_DONE 2u
#define DP_SPIN_DEFAULT (1u << 21) /* polls of about a microsecond each: seconds */

DP_FN uint32_t dp_expert_words(uint32_t first_tile) { return DP_WORDS_PER_TILE * first_tile; }
/* may a DOWN item of the expert start, given the value it read from word 0 */
DP_FN int dp_down_ready(uint32_t glu_done, uint32_t glu_items) { return glu_done >= glu_items; }
/* is the item whose add to word 2 returned `items_done_before` the expert's last */
DP_FN int dp_is_last(uint32_t items_done_before, uint32_t glu_items, uint32_t down_items) {
    return items_done_before + 1u == glu_items + down_items;
}
DP_FN uint32_t dp_spin_limit(uint32_t reserved) { return reserved ? reserved : DP_SPIN_DEFAULT; }

#endif
