// Arrival protocol of the K split (plain C, host and device): how the workgroups that share one output tile find
// out which of them is the last to have written its partial sums.
//
// One 32-bit word per output tile lives in the caller's workspace: (tag << 8) | count.  `tag` (24 bits, never 0)
// names the launch; `count` is the number of slices of THAT launch that have arrived.  A slice replaces the word
// by splitk_arrive(word) with a compare-and-swap and learns how many slices arrived before it.  A word that carries
// another launch's tag, or a count that no slice of this launch can have left (>= splits), is left over from a
// launch that never finished (killed, aborted) or from uninitialised memory: it counts as "nobody has arrived",
// so a poisoned word cannot make a tile wait for slices that will never come or be skipped by all of them.
// The last slice stores 0 when it has read the others' sums, so that a replay of a captured launch (which carries
// the same tag again) starts from a clean word.
#ifndef I8F_SPLITK_PROTOCOL_H
#define I8F_SPLITK_PROTOCOL_H

#include <stdint.h>

#if defined(__HIPCC__) || defined(__CUDACC__)
#define I8F_HD __host__ __device__
#else
#define I8F_HD
#endif

#define I8F_SPLITK_MAX_SPLITS 255u

// -> the word to store; *arrived_before = slices of this launch that had arrived already (0 .. splits - 1)
I8F_HD static inline uint32_t splitk_arrive(uint32_t word, uint32_t tag, uint32_t splits, uint32_t *arrived_before) {
    const uint32_t count = word & 0xffu, wtag = word >> 8;
    if (wtag == tag && count >= 1u && count < splits) {
        *arrived_before = count;
        return word + 1u;
    }
    *arrived_before = 0u;
    return (tag << 8) | 1u;
}

// the tag of the n-th launch of a process (n = 0, 1, ...): 24 bits, never 0
I8F_HD static inline uint32_t splitk_tag(uint32_t n) { return n % 0xffffffu + 1u; }

#endif
