// ft_launch_plan.hpp -- how work that needs more workgroups than one launch may hold is cut into
// launches. Plain host arithmetic (no HIP types), so that it can be tested without a GPU.
#pragma once

#include <stdint.h>

namespace fth {

// Piece `index` of `workgroups` workgroups cut into launches of at most `limit` each: every piece but
// the last is full, piece k starts at workgroup k * limit. Returns false when `index` lies behind the
// last piece (so: for (k = 0; plan_launch_piece(total, limit, k, &first, &count); ++k) launch).
inline bool plan_launch_piece(uint64_t workgroups, uint64_t limit, uint64_t index, uint64_t* first, uint64_t* count)
{
    if (limit == 0) return false;
    const uint64_t begin = index * limit;
    if (index != 0 && begin / index != limit) return false;  // overflow: far behind the last piece
    if (begin >= workgroups) return false;
    *first = begin;
    *count = workgroups - begin < limit ? workgroups - begin : limit;
    return true;
}

inline uint64_t launch_piece_count(uint64_t workgroups, uint64_t limit)
{
    return limit == 0 ? 0 : workgroups / limit + (workgroups % limit != 0 ? 1 : 0);
}

// Batches of the many-segment launch: a batch holds at most `max_segs` segments and `max_wgs`
// workgroups and is filled in order. True when a batch that holds `count` segments and `used`
// workgroups has to be launched before a segment of `wgs` workgroups can join.
inline bool segment_batch_is_full(int count, uint64_t used, uint64_t wgs, int max_segs, uint64_t max_wgs)
{
    return count == max_segs || (count > 0 && used + wgs > max_wgs);
}

// The same rule over a whole list: segment i needs wgs[i] workgroups (each at most `max_wgs`). Writes
// the batch index of every segment and returns the number of batches.
inline int plan_segment_batches(const uint64_t* wgs, int n, int max_segs, uint64_t max_wgs, int* batch_of)
{
    int batch = 0, count = 0;
    uint64_t used = 0;
    for (int i = 0; i < n; ++i) {
        if (segment_batch_is_full(count, used, wgs[i], max_segs, max_wgs)) {
            ++batch;
            count = 0;
            used = 0;
        }
        batch_of[i] = batch;
        ++count;
        used += wgs[i];
    }
    return n > 0 ? batch + 1 : 0;
}

}  // namespace fth
