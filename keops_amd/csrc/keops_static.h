// Interface between the host library (keops_hip.cpp, host compiler) and the device code that is compiled into
// libkeops_hip.so itself (keops_static.hip, hipcc).
#pragma once
#include <stddef.h>

// Size of the static device scratch buffer behind keops_hip_launch_noalloc: 128 MiB per GPU, held from the first
// use of the library's device code on that GPU until the process ends.
#define KEOPS_STATIC_SCRATCH_BYTES (128u << 20)

int keops_static_scratch(int device, void** ptr, size_t* bytes);
int keops_static_fill_zero(void* dst, size_t bytes, void* stream);
// n elements: IEEE half -> float (to_float != 0) or float -> half (round to nearest even)
int keops_static_convert_half(void* dst, const void* src, long long n, int to_float, void* stream);

// Lookup table of a block-sparse launch built on the device (no read-back of the ranges): see keops_static.hip.
struct KeopsRangeBuild {
  const long long *rx, *sl, *ry;  // the caller's row ranges [nranges][2], slices [nranges], reduced ranges [nred][2]
  long long nranges, nred, rows_total, cols_total, rows_per_block, nblocks_max;
  long long *lookup;              // out: [nblocks_max][3] (range id, first row, end row); unused entries are empty
  long long *sl_clean, *ry_clean; // out: copies of sl / ry with every index clamped to its axis
  long long *nb, *work, *order, *offs;  // work arrays [nranges] each
  unsigned *status;               // out, host memory mapped into the device, never cleared here: [0] = 1 an index was out of
                                  // bounds (clamped), [1] = 1 more workgroups than nblocks_max
};
// number of long long words the arrays above take (lookup, sl_clean, ry_clean, nb, work, order, offs, status)
size_t keops_static_range_build_words(long long nranges, long long nred, long long nblocks_max);
int keops_static_build_ranges(const KeopsRangeBuild* b, void* stream);
