#include "planner.h"

#include <cstddef>
#include <limits>

namespace dnnc {

PoolSimulator::PoolSimulator() { holes_.push_back({0, std::numeric_limits<int64_t>::max() - 1}); }

int64_t PoolSimulator::round_size(int64_t bytes) { return bytes <= 0 ? 0 : ((bytes - 1) / 32 + 1) * 32; }

void PoolSimulator::note_peak() {
  if (holes_.back().lo > peak_) peak_ = holes_.back().lo;
}

int64_t PoolSimulator::reserve(int64_t id, int64_t size) {
  // First fit.  With inclusive bounds hi - lo is one less than the hole's
  // length, so the comparison demands a hole strictly larger than `size`.
  size_t h = 0;
  while (h < holes_.size() && holes_[h].hi - holes_[h].lo < size) h++;
  if (h == holes_.size()) return -1;  // cannot happen: the last hole is unbounded
  const int64_t lo = holes_[h].lo;
  const Live blk{id, lo, lo + size - 1};
  // Keep live_ ordered by start: the new block goes before the first entry
  // that does not start below it.
  size_t at = 0;
  while (at < live_.size() && live_[at].lo < lo) at++;
  live_.insert(live_.begin() + (long)at, blk);
  holes_[h].lo += size;
  note_peak();
  return lo;
}

bool PoolSimulator::release(int64_t id) {
  size_t a = 0;
  while (a < live_.size() && live_[a].id != id) a++;
  if (a == live_.size()) return false;
  const Live blk = live_[a];
  live_.erase(live_.begin() + (long)a);

  // Merge with the first hole that touches the block on either side.
  for (size_t h = 0; h < holes_.size(); h++) {
    if (holes_[h].hi == blk.lo - 1) {          // hole ends where the block starts
      holes_[h].hi = blk.hi;
      if (h + 1 < holes_.size() && holes_[h + 1].lo == holes_[h].hi + 1) {
        holes_[h + 1].lo = holes_[h].lo;       // bridged two holes
        holes_.erase(holes_.begin() + (long)h);
      }
      note_peak();
      return true;
    }
    if (holes_[h].lo == blk.hi + 1) {          // hole starts where the block ends
      holes_[h].lo = blk.lo;
      if (h > 0 && holes_[h - 1].hi == holes_[h].lo - 1) {
        holes_[h - 1].hi = holes_[h].hi;
        holes_.erase(holes_.begin() + (long)h);
      }
      note_peak();
      return true;
    }
  }
  // No neighbour is free: a new hole, kept in address order.
  for (size_t h = 0; h < holes_.size(); h++) {
    if (holes_[h].lo > blk.hi) {
      holes_.insert(holes_.begin() + (long)h, Hole{blk.lo, blk.hi});
      note_peak();
      return true;
    }
    if (h + 1 == holes_.size() && holes_[h].lo < blk.hi) {
      holes_.push_back(Hole{blk.lo, blk.hi});
      note_peak();
      return true;
    }
  }
  return false;
}

std::vector<std::pair<int64_t, int64_t>> PoolSimulator::free_list() const {
  std::vector<std::pair<int64_t, int64_t>> out;
  for (const Hole &h : holes_) out.push_back({h.lo, h.hi});
  return out;
}

}  // namespace dnnc
