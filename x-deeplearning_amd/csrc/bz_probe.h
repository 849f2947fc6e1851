// bz_probe.h -- measurement aids exported by the library but not part of its public interface (include/blaze_hip.h):
// kernels that isolate one access pattern of the pooling kernel so that its share of a launch can be timed and
// counted on its own (bench.py --gather-probe).
#pragma once

#include "blaze_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Measurement aid, no counterpart in the reference: a pure random gather of 64- or 128-byte rows, the access pattern
 * of the pooling kernel with everything else taken away.  `groups` lane groups (one lane per 16-byte chunk of a row)
 * each read `rows_per_group` (1, 4, 8 or 16) rows at hashed positions of `region` (16-byte aligned; all loads of a
 * group are issued before the first is used), fold them and write one row to sink[group].  With `side` not NULL every
 * row read is accompanied by the read of the 4-byte word side[row] (the per-row scale of an int8 table kept in an array
 * of its own).  The caller times the launch; bytes read = groups * rows_per_group * (row_bytes [+ 4]).
 * Row of load r of group g, 32-bit arithmetic: h = (g * rows_per_group + r) * 2654435761 + seed; h ^= h >> 15;
 * h *= 2246822519; h ^= h >> 13; row = (h * rows) >> 32 with rows = region_bytes / row_bytes.
 */
BZ_API int bz_probe_gather(const void* region, int64_t region_bytes, int row_bytes, const float* side, void* sink,
                           int64_t groups, int rows_per_group, uint32_t seed, bz_stream_t stream);

#ifdef __cplusplus
}
#endif
