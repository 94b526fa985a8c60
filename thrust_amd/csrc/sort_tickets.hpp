// Which tile a workgroup of a radix-sort pass takes.  Plain C++ (also compiled for the host by
// tests/cpp/test_sort_tickets.cpp, which checks the properties stated below for every tile count).
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define TA_TICKETS_FN __host__ __device__ inline
#else
#define TA_TICKETS_FN inline
#endif

namespace ta {

// The digit runs of tile t + 1 continue those of tile t in memory, and the cache line in which
// one ends and the other begins is written in part by both.  When both tiles run on the same
// XCD the two parts meet in that XCD's L2 and leave as one line; otherwise each costs a
// partial-line write to memory -- for 288-byte runs a third of a pass (a kernel with nothing
// but a pass's memory accesses: 0.60 ms, 0.54 ms with neighbouring tiles on one XCD).
// Workgroups go to the XCDs in turn (workgroup i to XCD i % 8), so the workgroups of class
// k = i % 8 draw their tickets from a counter of their own and ticket c of class k stands for
// tile class_tile(k, c): 8 consecutive tiles, then the 8 tiles 64 further on, ...; the tiles
// past the last whole group of 64 are dealt to the classes in order, each as many as it has
// workgroups left.  With exactly `tiles` workgroups every tile is taken exactly once whatever
// the hardware does; inside a class tiles are taken in rising order.  (Groups of 2 / 4 / 8 / 16 /
// 32 tiles: 0.545 / 0.509 / 0.495 / 0.540 / 0.596 ms per pass over 2^28 uint32 keys; one counter for
// all: 0.576 ms.)
constexpr uint32_t TILES_PER_GROUP = 8;
constexpr uint32_t TICKET_CLASSES = 8;
constexpr uint32_t TICKET_STRIDE = 32;  // words between the counters of two classes: a cache line each

TA_TICKETS_FN uint32_t class_tile(uint32_t k, uint32_t c, uint32_t tiles) {
  constexpr uint32_t G = TILES_PER_GROUP, S = TICKET_CLASSES * G;
  const uint32_t whole = tiles / S;  // groups of 64 tiles that are complete
  if (c < whole * G) return ((c / G) * TICKET_CLASSES + k) * G + c % G;
  // class k has tiles / 8 workgroups, one more if k < tiles % 8; `rest` of them are past the whole groups
  const uint32_t rest = tiles / TICKET_CLASSES - whole * G, extra = tiles % TICKET_CLASSES;
  const uint32_t before = k * rest + (k < extra ? k : extra);  // tail tiles of the classes before k
  return whole * S + before + (c - whole * G);
}

}  // namespace ta
