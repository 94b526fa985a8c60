// Host-side check of the rule by which the workgroups of a radix-sort pass take their tiles
// (thrust_amd/csrc/sort_tickets.hpp, the very function the kernel calls):
//   1. with `tiles` workgroups, workgroup i drawing the next ticket of class i % 8, every tile
//      is taken exactly once and the tiles of a class rise with its tickets -- for every tile
//      count up to 20000 and a few large ones;
//   2. no schedule of two dispatcher models leaves the pass stuck.  A tile can finish once every
//      lower tile has been taken (its look-back then finds their counts).  Model A: the
//      workgroups of class k run on XCD k only, each XCD dispatching its own in order at its own
//      pace into any number of slots.  Model B: workgroups are dispatched in order of their index
//      into at least 64 slots anywhere.  Random paces and finishing orders, many seeds.
#include <cstdint>
#include <cstdio>
#include <random>
#include <vector>

#include "../../thrust_amd/csrc/sort_tickets.hpp"

using ta::class_tile;

static bool bijection(uint32_t tiles) {
  std::vector<uint8_t> seen(tiles, 0);
  uint32_t next[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  int64_t last[8] = {-1, -1, -1, -1, -1, -1, -1, -1};
  for (uint32_t i = 0; i < tiles; ++i) {
    const uint32_t k = i % 8, t = class_tile(k, next[k]++, tiles);
    if (t >= tiles || seen[t]) return false;
    if ((int64_t)t <= last[k]) return false;
    last[k] = t;
    seen[t] = 1;
  }
  return true;
}

// One run of a dispatcher model; false when it gets stuck.
static bool finishes(uint32_t tiles, bool bound_to_xcd, uint32_t slots_per_xcd, uint32_t seed) {
  std::mt19937 rnd(seed);
  std::vector<uint8_t> taken(tiles, 0);
  uint32_t next_ticket[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  uint32_t next_of_class[8] = {0, 1, 2, 3, 4, 5, 6, 7};  // model A: next workgroup index of each XCD
  uint32_t next_index = 0;                                // model B
  std::vector<std::vector<uint32_t>> resident(8);
  uint32_t lowest_untaken = 0, finished = 0;
  auto take = [&](uint32_t i) {
    const uint32_t k = i % 8, t = class_tile(k, next_ticket[k]++, tiles);
    taken[t] = 1;
    return t;
  };
  while (finished < tiles) {
    bool could_dispatch = false, could_finish = false, moved = false;
    if (bound_to_xcd) {
      for (uint32_t x = 0; x < 8; ++x)
        while (resident[x].size() < slots_per_xcd && next_of_class[x] < tiles) {
          could_dispatch = true;
          if (rnd() % 4 == 0) break;  // this XCD falls behind for a while
          resident[x].push_back(take(next_of_class[x]));
          next_of_class[x] += 8;
          moved = true;
        }
    } else {
      while (next_index < tiles) {
        std::vector<uint32_t> room;
        for (uint32_t x = 0; x < 8; ++x)
          if (resident[x].size() < slots_per_xcd) room.push_back(x);
        if (room.empty()) break;
        could_dispatch = true;
        if (rnd() % 8 == 0) break;
        resident[room[rnd() % room.size()]].push_back(take(next_index++));
        moved = true;
      }
    }
    while (lowest_untaken < tiles && taken[lowest_untaken]) ++lowest_untaken;
    for (uint32_t x = 0; x < 8; ++x) {
      std::vector<uint32_t> keep;
      for (uint32_t t : resident[x]) {
        if (t < lowest_untaken) {  // every lower tile is taken
          could_finish = true;
          if (rnd() % 3 != 0) {
            ++finished;
            moved = true;
            continue;
          }
        }
        keep.push_back(t);
      }
      resident[x].swap(keep);
    }
    if (!moved && !could_dispatch && !could_finish) return false;  // nothing can ever move again
  }
  return true;
}

int main() {
  for (uint32_t tiles = 1; tiles <= 20000; ++tiles)
    if (!bijection(tiles)) {
      std::printf("tiles=%u: not every tile exactly once, or not rising inside a class\n", tiles);
      return 1;
    }
  for (uint32_t tiles : {65535u, 65536u, 65537u, 1u << 20, (1u << 20) + 13u, 3000001u})
    if (!bijection(tiles)) {
      std::printf("tiles=%u: not every tile exactly once, or not rising inside a class\n", tiles);
      return 1;
    }
  const uint32_t counts[] = {1, 7, 8, 9, 63, 64, 65, 127, 500, 513, 1000, 4097, 14564};
  for (uint32_t tiles : counts)
    for (uint32_t seed = 1; seed <= 8; ++seed) {
      for (uint32_t slots : {1u, 2u, 3u, 64u})  // per XCD
        if (!finishes(tiles, true, slots, seed)) {
          std::printf("stuck: tiles=%u bound to XCDs, %u slots per XCD, seed %u\n", tiles, slots, seed);
          return 1;
        }
      for (uint32_t slots : {8u, 16u, 64u})  // per XCD: 64, 128, 512 in all
        if (!finishes(tiles, false, slots, seed)) {
          std::printf("stuck: tiles=%u dispatched in order, %u slots, seed %u\n", tiles, 8 * slots, seed);
          return 1;
        }
    }
  std::printf("PASSED\n");
  return 0;
}
