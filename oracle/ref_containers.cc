// TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// C entry points over the reference's own header-only containers, compiled in
// place from the reference tree (never copied): common/skip_list.h,
// common/parallel_skip_list.h and the mixer in common/utils.h. Used to check
// the plain-C restatement of the same containers and, optionally, as a timed
// CPU baseline for id -> row lookup.
#include <cstdint>
#include <ctime>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "common/parallel_skip_list.h"
#include "common/utils.h"

namespace {
struct Row {
  std::vector<float> val;
};
using Map = kraken::ParallelSkipList<uint64_t, Row>;
}  // namespace

extern "C" {

uint64_t ref_hash64(uint64_t v) { return kraken::utils::Hash(v); }
uint64_t ref_hash64_pair(uint64_t a, uint64_t b) { return kraken::utils::Hash(a, b); }

void* ref_map_create() { return new Map(); }
void ref_map_destroy(void* m) { delete static_cast<Map*>(m); }
uint64_t ref_map_hit_slot(void* m, uint64_t id) { return static_cast<Map*>(m)->HitSlot(id); }

// Insert rows [n, dim]; returns how many keys were new.
int64_t ref_map_insert(void* m, const uint64_t* ids, int64_t n, const float* vals, int64_t dim) {
  Map* map = static_cast<Map*>(m);
  int64_t fresh = 0;
  for (int64_t i = 0; i < n; ++i) {
    Row r;
    r.val.assign(vals + i * dim, vals + (i + 1) * dim);
    fresh += map->Insert(ids[i], r) ? 1 : 0;
  }
  return fresh;
}

// hit[i] = 1 and out[i, :] = row when present, else hit[i] = 0.
void ref_map_find(void* m, const uint64_t* ids, int64_t n, uint8_t* hit, float* out, int64_t dim) {
  Map* map = static_cast<Map*>(m);
  for (int64_t i = 0; i < n; ++i) {
    auto h = map->UniqueSkipListHandler(map->HitSlot(ids[i]));
    auto it = h.skip_list.Find(ids[i]);
    hit[i] = it.Valid() ? 1 : 0;
    if (it.Valid() && out) {
      const Row& r = it.value();
      for (int64_t j = 0; j < dim; ++j) out[i * dim + j] = r.val[j];
    }
  }
}

// The clean-up walk of ps/ps.cc:92-109 with the routing decision replaced by a list of ids to
// drop: every slot under its unique handler, SkipList::Remove on the rows that go. Returns how
// many rows were removed.
int64_t ref_map_erase(void* m, const uint64_t* ids, int64_t n) {
  Map* map = static_cast<Map*>(m);
  std::unordered_map<uint64_t, bool> drop;
  for (int64_t i = 0; i < n; ++i) drop[ids[i]] = true;
  int64_t removed = 0;
  for (size_t s = 0; s < map->slot_count(); ++s) {
    auto h = map->UniqueSkipListHandler(s);
    auto it = h.skip_list.Begin();
    while (it.Valid()) {
      if (drop.count(it.key())) {
        it = h.skip_list.Remove(it);
        ++removed;
      } else {
        it.Next();
      }
    }
  }
  return removed;
}

// Keys in slot-major, key-ascending order (the order the checkpoint writer walks).
int64_t ref_map_keys(void* m, uint64_t* ids) {
  Map* map = static_cast<Map*>(m);
  int64_t k = 0;
  for (size_t s = 0; s < map->slot_count(); ++s) {
    auto h = map->SharedSkipListHandler(s);
    for (auto it = h.skip_list.Begin(); it.Valid(); it.Next()) ids[k++] = it.key();
  }
  return k;
}

}  // extern "C"
