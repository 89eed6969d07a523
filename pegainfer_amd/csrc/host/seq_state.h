// Per-request recurrent state beside the paged key/value cache: every request slot owns one contiguous fp32 region of a
// device arena; the layers of a model reserve their parts of that region once, at configuration time (convolution tails,
// matrix memories, normaliser vectors, running maxima).  Pure host bookkeeping: the arena's memory belongs to the runtime
// that uses the layout, kernels get  base + part offset  and add  slot * floats_per_slot  themselves.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

namespace pq {

class StateLayout {
 public:
  // reserves `floats` values for a named part of every slot's region; returns the part's offset inside the region
  int64_t reserve(const std::string& what, int64_t floats) {
    const int64_t at = total_;
    parts_.push_back({what, at, floats});
    total_ += floats;
    return at;
  }
  int64_t floats_per_slot() const { return total_; }
  size_t parts() const { return parts_.size(); }

 private:
  struct Part { std::string what; int64_t offset, floats; };
  std::vector<Part> parts_;
  int64_t total_ = 0;
};

}  // namespace pq
