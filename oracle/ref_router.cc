// Test infrastructure only. Builds the reference's own consistent-hash ring (common/router.cc,
// compiled where it lies) and asks it who owns rows, so that the routing rule the table hooks
// restate -- Router::Hit(utils::Hash(table_id, sparse_id)), as ps/ps.cc:100 and :306 call it --
// is pinned by the code that defines it.
//
//   ref_router <table_id> <n_ids> <node name> [<node name> ...]
//
// Nodes get the ids 0, 1, 2, ... in the order given (Router::Add wants them ascending). Output:
//   vnode <hash_v> <node_id>      one line per virtual node, ascending hash (the ring)
//   id <sparse_id> <owner>        for sparse_id = splitmix64(r), r = 0 .. n_ids - 1, and for a
//                                 few ids picked to fall on and around the ring's ends
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <string>

#include "common/router.h"
#include "common/utils.h"

using namespace kraken;

static uint64_t splitmix64(uint64_t x) {
  uint64_t z = x + 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

int main(int argc, char** argv) {
  if (argc < 4) {
    fprintf(stderr, "usage: see the head of oracle/ref_router.cc\n");
    return 1;
  }
  const uint64_t table_id = strtoull(argv[1], nullptr, 10);
  const int64_t n = atoll(argv[2]);
  Router router;
  for (int i = 3; i < argc; ++i) {
    if (!router.Add((uint64_t)(i - 3), argv[i])) return 2;
  }
  for (const auto& v : router.vnodes()) printf("vnode %" PRIu64 " %" PRIu64 "\n", v.hash_v, v.node_id);
  for (int64_t r = 0; r < n; ++r) {
    const uint64_t id = splitmix64((uint64_t)r);
    printf("id %" PRIu64 " %" PRIu64 "\n", id, router.Hit(utils::Hash(table_id, id)));
  }
  for (uint64_t id : {0ull, 1ull, ~0ull, ~0ull - 1, 1ull << 63})
    printf("id %" PRIu64 " %" PRIu64 "\n", id, router.Hit(utils::Hash(table_id, id)));
  // raw ring look-ups on and next to every virtual node, and at both ends of the hash space
  for (const auto& v : router.vnodes()) {
    for (uint64_t hv : {v.hash_v - 1, v.hash_v, v.hash_v + 1})
      printf("hit %" PRIu64 " %" PRIu64 "\n", hv, router.Hit(hv));
  }
  for (uint64_t hv : {0ull, ~0ull}) printf("hit %" PRIu64 " %" PRIu64 "\n", hv, router.Hit(hv));
  return 0;
}
