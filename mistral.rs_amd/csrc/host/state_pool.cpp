// state_pool.cpp -- host bookkeeping of fixed-size per-sequence state slots (C++, no device code): the slots that recurrent mixers (short-convolution taps, state-space
// states) keep per live sequence, next to the paged K / V blocks of the attention layers.  Role of `RecurrentStatePool`'s free list in the reference
// (mistralrs-core/src/kv_cache/hybrid_cache.rs:76-410: allocate / free / num_free_slots / capacity); the device tensors [slots, ...] belong to the model, which treats a slot
// whose sequence starts at position 0 as zero, so a freed slot needs no clearing before it is handed out again.
// Slots are handed out lowest-free-first and a freed slot is the next one out (LIFO), so reuse happens as early as possible.  Not thread safe (one engine thread per rank).
#include <stddef.h>
#include <stdint.h>

#include <unordered_map>
#include <vector>

namespace mrs_host {
struct StatePool {
  std::vector<int64_t> free_list;                  // back = next out
  std::unordered_map<uint64_t, int64_t> owner;     // request id -> slot
  size_t capacity = 0;
};
}  // namespace mrs_host
using mrs_host::StatePool;

extern "C" {
void *mrs_state_pool_create(size_t num_slots) {
  if (num_slots == 0) return nullptr;
  auto *p = new StatePool;
  p->capacity = num_slots;
  for (size_t i = num_slots; i-- > 0;) p->free_list.push_back((int64_t)i);
  return p;
}
void mrs_state_pool_destroy(void *h) { delete (StatePool *)h; }
size_t mrs_state_pool_capacity(void *h) { return ((StatePool *)h)->capacity; }
size_t mrs_state_pool_num_free_slots(void *h) { return ((StatePool *)h)->free_list.size(); }
/* the request's slot (allocated on first use); -1 = no slot free */
int64_t mrs_state_pool_allocate(void *h, uint64_t request_id) {
  auto *p = (StatePool *)h;
  auto it = p->owner.find(request_id);
  if (it != p->owner.end()) return it->second;
  if (p->free_list.empty()) return -1;
  const int64_t s = p->free_list.back();
  p->free_list.pop_back();
  p->owner.emplace(request_id, s);
  return s;
}
/* -1 = the request holds no slot */
int64_t mrs_state_pool_slot_of(void *h, uint64_t request_id) {
  auto *p = (StatePool *)h;
  auto it = p->owner.find(request_id);
  return it == p->owner.end() ? -1 : it->second;
}
void mrs_state_pool_free(void *h, uint64_t request_id) {
  auto *p = (StatePool *)h;
  auto it = p->owner.find(request_id);
  if (it == p->owner.end()) return;
  p->free_list.push_back(it->second);
  p->owner.erase(it);
}
}
