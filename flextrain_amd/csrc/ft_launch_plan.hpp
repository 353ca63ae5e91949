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

// Where the tiles of a step start when its arrays do not reach their vector alignment together.
// One array per entry: its address, its element size (2 or 4 bytes) and a weight (bytes moved per
// element, written bytes counted twice: a store that covers part of a cache line costs more than a
// load that does). Tiles are 256 elements, so a choice of `head` elements in front of the first
// tile fixes, for every array, whether its tiles start on 128-byte lines (whole-line traffic) and
// whether its 4-element units are aligned as vectors. Returns the head below 64 (the period of a
// 2-byte array's line phase) with the largest weighted score, the smallest such on a tie, and the
// set of arrays whose tiles then start on lines (bit k: array k).
struct ArrayPlacement {
    uint64_t address;
    uint32_t elem_bytes;
    uint32_t weight;
};
constexpr uint32_t kLineBytes = 128;
constexpr uint32_t kRelaxedHeadPeriod = 64;

inline uint32_t plan_relaxed_head(const ArrayPlacement* arrays, int count, uint32_t* on_lines)
{
    uint32_t best_head = 0, best_mask = 0;
    uint64_t best_score = 0;
    for (uint32_t head = 0; head < kRelaxedHeadPeriod; ++head) {
        uint64_t score = 0;
        uint32_t mask = 0;
        for (int k = 0; k < count; ++k) {
            const uint64_t at = arrays[k].address + static_cast<uint64_t>(head) * arrays[k].elem_bytes;
            if (at % kLineBytes == 0) {
                score += 4ull * arrays[k].weight;
                mask |= 1u << k;
            } else if (at % (4ull * arrays[k].elem_bytes) == 0) {
                score += arrays[k].weight;
            }
        }
        if (head == 0 || score > best_score) {
            best_head = head;
            best_score = score;
            best_mask = mask;
        }
    }
    *on_lines = best_mask;
    return best_head;
}

}  // namespace fth
