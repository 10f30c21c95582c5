// Memory-pool planner: replays a program's malloc/dealloc events through an
// address-space simulator and returns one byte offset per tensor plus the pool
// size.  Behaviour follows the reference planner bit for bit
// (src/Transform/DNN/mallocPoolOpt.hpp:21-140, 212-218), including its
// inclusive-end fit rule under which a hole of exactly the requested size is
// NOT reused, its handling of zero-byte tensors, and "pool size = highest
// start of the trailing free block ever seen".
#pragma once
#include <cstdint>
#include <vector>

namespace dnnc {

class PoolSimulator {
 public:
  PoolSimulator();
  // prod(shape) * element bytes -> bytes the planner reserves (multiple of 32)
  static int64_t round_size(int64_t bytes);
  // Reserves `size` (already rounded) bytes for tensor `id`; returns its offset.
  int64_t reserve(int64_t id, int64_t size);
  // Returns tensor `id`'s bytes to the free list; false if it is not live.
  bool release(int64_t id);
  int64_t peak() const { return peak_; }
  // free list as (first byte, last byte) pairs, for tests
  std::vector<std::pair<int64_t, int64_t>> free_list() const;

 private:
  struct Hole { int64_t lo, hi; };            // inclusive
  struct Live { int64_t id, lo, hi; };        // inclusive; hi = lo - 1 for empty tensors
  std::vector<Hole> holes_;                   // ascending
  std::vector<Live> live_;                    // ascending by lo
  int64_t peak_ = 0;
  void note_peak();
};

}  // namespace dnnc
