// Set-up time building blocks shared by the format builders and the plan (sort.hip): a stable radix sort of
// (key, 32-bit payload) pairs and an exclusive scan, hand-written for gfx950.
#pragma once

#include "common.h"

namespace gnnagg {

// Stable ascending sort of n pairs by the low `bits` bits of the key, 8 bits a pass, ping-pong between the (a) and
// (b) arrays: the input is in (key_a, val_a); *result_in_b says where the sorted pairs ended up.  `workspace`:
// sort_pairs_workspace_bytes(n) bytes of device memory (the histograms), 256-byte aligned -- the call then only
// enqueues on `st`; nullptr: the call allocates them and synchronises `st` before it returns.
size_t sort_pairs_workspace_bytes(int64_t n);
int sort_pairs_u64(uint64_t *key_a, uint64_t *key_b, uint32_t *val_a, uint32_t *val_b, int64_t n, int bits,
                   hipStream_t st, bool *result_in_b, void *workspace = nullptr);
int sort_pairs_u32(uint32_t *key_a, uint32_t *key_b, uint32_t *val_a, uint32_t *val_b, int64_t n, int bits,
                   hipStream_t st, bool *result_in_b, void *workspace = nullptr);

// out[i] = in[0] + ... + in[i - 1] for sums below 2^32 (in == out is fine).  Synchronises `st` before it returns.
int exclusive_scan_u32(const uint32_t *in, uint32_t *out, int64_t n, hipStream_t st);

}  // namespace gnnagg
