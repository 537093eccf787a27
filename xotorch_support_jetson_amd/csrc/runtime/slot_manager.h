// State slots of models with recurrent layers: one slot per live request in a pool of fixed size, handed out on
// admission (lowest free slot first, so a small pool is reused at once) and returned when the request ends.  The
// device-side state of a slot (models.transformer.StatePool) is cleared by the runner when the slot is handed out.
// Not internally synchronised: each engine drives it from its single executor thread, like the block manager.
#pragma once
#include <algorithm>
#include <cstdint>
#include <functional>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

namespace xot_rt {

class SlotManager {
 public:
  explicit SlotManager(int64_t slots) : slots_(slots) {
    if (slots <= 0) throw std::invalid_argument("slots must be > 0");
    for (int64_t s = 0; s < slots; ++s) free_.push_back((int32_t)s);
    std::make_heap(free_.begin(), free_.end(), std::greater<int32_t>());  // min-heap: lowest slot on top
  }
  int64_t slots() const { return slots_; }
  int64_t num_free() const { return (int64_t)free_.size(); }
  bool has(const std::string& rid) const { return of_.count(rid) != 0; }
  int64_t slot(const std::string& rid) const {
    auto it = of_.find(rid);
    if (it == of_.end()) throw std::out_of_range("no state slot for request " + rid);
    return it->second;
  }
  int64_t acquire(const std::string& rid) {
    if (of_.count(rid)) throw std::invalid_argument("request " + rid + " already holds a state slot");
    if (free_.empty())
      throw std::runtime_error("state slots exhausted: all " + std::to_string(slots_) + " are held by live requests");
    std::pop_heap(free_.begin(), free_.end(), std::greater<int32_t>());
    const int32_t s = free_.back();
    free_.pop_back();
    of_[rid] = s;
    return s;
  }
  void release(const std::string& rid) {
    auto it = of_.find(rid);
    if (it == of_.end()) return;
    free_.push_back(it->second);
    std::push_heap(free_.begin(), free_.end(), std::greater<int32_t>());
    of_.erase(it);
  }

 private:
  int64_t slots_;
  std::vector<int32_t> free_;
  std::unordered_map<std::string, int32_t> of_;
};

}  // namespace xot_rt
