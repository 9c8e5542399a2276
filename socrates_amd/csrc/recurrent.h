// What the recurrences with a matrix state per head share: the size of a batch of tokens, the
// barrier for threads that meet in LDS only, the dispatch by state size, and how many of a head's
// columns one workgroup owns.
#pragma once

#include "common.h"

// (tokens per batch: 16 for states of up to 64 keys, else 8: what LDS holds twice over)
constexpr int rec_batch(int keys) { return keys <= 64 ? 16 : 8; }

// A barrier for threads that meet in LDS only: a wave waits for its own LDS accesses, not for its global
// loads and stores in flight (__syncthreads waits for those too, which would drain the next batch's
// loads, issued on purpose before the current batch is computed, at every barrier).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

#define SOC_BY_STATE_SIZE(D, CALL)                                         \
    switch (((D) + 15) / 16) {                                              \
        case 1: CALL(16); break;   case 2: CALL(32); break;                 \
        case 3: CALL(48); break;   case 4: CALL(64); break;                 \
        case 5: case 6: CALL(96); break;                                    \
        case 7: case 8: CALL(128); break;                                   \
        case 9: case 10: case 11: case 12: CALL(192); break;                \
        case 13: case 14: case 15: case 16: CALL(256); break;               \
        default: return (int)hipErrorInvalidValue;                          \
    }

// Columns per workgroup: 64, or 16 where heads and sequences alone leave most compute units idle.
// (A step with a prompt portion in it is as long as that portion's walk, whatever else is in the step.)
static int columns_per_workgroup(int H, int cols, int n_seqs, int max_q_len) {
    if (max_q_len > 64) return 16;
    return (long long)H * ((cols + 63) / 64) * n_seqs >= 192 ? 64 : 16;
}

