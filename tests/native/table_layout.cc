// table_layout.cc -- the host side of the chunk tables (context.cc: count_chunks, fill_chunks, xcd_chunk /
// xcd_slot, line_slot, table_slots, xcd_order) checked without a GPU: every chunk of every segment
// appears exactly once, at the table entry that its workgroup reads, the padding entries are empty,
// the four workgroups of one XCD in a group of 32 read one 128-byte line, and each XCD walks runs of
// consecutive chunks.  Prints "table layout ok".
#include <cstdio>
#include <cstdlib>
#include <map>
#include <random>
#include <vector>

#include "internal.h"

using namespace hvdhip;

// context.cc calls into the two translation units that hold kernels; this test links without them.
void hvdhip::copy_cache_forget_stream(hipStream_t) {}
void hvdhip::adasum_forget_stream(hipStream_t) {}

#define REQUIRE(cond)                                                 \
  do {                                                                \
    if (!(cond)) {                                                    \
      std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);     \
      std::exit(1);                                                   \
    }                                                                 \
  } while (0)

static void check(const std::vector<Seg>& segs, uint32_t chunk_units, uint32_t tes, uint32_t bes) {
  const uint64_t n = count_chunks(segs, chunk_units);
  REQUIRE(n != ~0ull);
  const uint64_t slots = table_slots(n);
  REQUIRE(slots % 32 == 0 && slots >= n && slots - n < 32);
  std::vector<Chunk> table(slots);
  for (auto& c : table) c = Chunk{~0ull, ~0ull, ~0ull, 0xffffffffu, 0xffffffffu};  // must all be overwritten
  fill_chunks(segs, chunk_units, tes, bes, table.data(), n);
  // what the workgroups of a launch of `slots` workgroups read, in workgroup order
  std::vector<Chunk> seen;
  uint64_t empty = 0;
  for (uint32_t b = 0; b < slots; ++b) {
    const uint32_t e = line_slot(b);
    REQUIRE(e < slots);
    REQUIRE((e & ~31u) == (b & ~31u));
    if (b + 8 < slots && (b & 31) < 24) REQUIRE(line_slot(b + 8) == e + 1);  // same XCD, next entry of the same line
    REQUIRE(e / 4 % 8 == b % 8);                                             // line number within the group = XCD
    const Chunk& c = table[e];
    REQUIRE(c.n != 0xffffffffu);
    if (c.n == 0) {
      REQUIRE(c.pad == 0);
      ++empty;
    } else {
      seen.push_back(c);
    }
  }
  REQUIRE(empty == slots - n && seen.size() == n);
  // every element of every segment exactly once, pads only at a segment's end
  std::map<uint64_t, uint64_t> covered;  // tensor address of a chunk -> elements
  for (const Chunk& c : seen) {
    REQUIRE(c.n <= chunk_units);
    REQUIRE(covered.emplace(c.tensor, c.n).second);
  }
  for (const Seg& s : segs) {
    uint64_t at = 0;
    while (at < s.n) {
      auto it = covered.find(s.tensor + at * tes);
      REQUIRE(it != covered.end());
      at += it->second;
    }
    REQUIRE(at == s.n);
  }
  uint64_t total = 0, pads = 0;
  for (const Chunk& c : seen) {
    total += c.n;
    pads += c.pad;
    REQUIRE(c.pad < 16);
  }
  uint64_t want_total = 0, want_pads = 0;
  for (const Seg& s : segs) {
    want_total += s.n;
    if (s.n) want_pads += (16 - (s.n * bes) % 16) % 16;
  }
  REQUIRE(total == want_total && pads == want_pads);
  // XCD order: workgroup b handles chunk xcd_chunk(b) of the natural order (tensor addresses ascend
  // with the natural order here), and xcd_slot is its inverse
  const uint32_t run = xcd_run(n, chunk_units * (tes > bes ? tes : bes));
  std::vector<uint64_t> natural;
  for (const Seg& s : segs)
    for (uint64_t st = 0; st < s.n; st += chunk_units) natural.push_back(s.tensor + st * tes);
  REQUIRE(natural.size() == n);
  for (uint64_t b = 0; b < n; ++b) {
    const uint64_t chunk = xcd_chunk(b, n, run);
    REQUIRE(chunk < n && xcd_slot(chunk, n, run) == b);
    REQUIRE(table[line_slot((uint32_t)b)].tensor == natural[chunk]);
  }
  // within a whole group of 8 * run chunks, XCD x (workgroups x, x + 8, ...) walks chunks x * run ... in order
  if (run > 1 && n >= 8ull * run) {
    for (uint32_t x = 0; x < 8; ++x)
      for (uint32_t i = 0; i + 1 < run; ++i)
        REQUIRE(xcd_chunk(x + 8ull * (i + 1), n, run) == xcd_chunk(x + 8ull * i, n, run) + 1);
  }
}

int main() {
  std::mt19937_64 rng(7);
  for (int rep = 0; rep < 300; ++rep) {
    const uint32_t tes = 1u << (rng() % 4), bes = (rep % 5 == 0 && tes == 4) ? 2 : tes;
    const uint32_t chunk_units = (rep % 3 ? 4096u : 65536u) / (tes > bes ? tes : bes);
    const int nseg = 1 + (int)(rng() % 40);
    std::vector<Seg> segs;
    uint64_t addr = 1 << 20, off = 0;
    for (int i = 0; i < nseg; ++i) {
      uint64_t n = rng() % 7 == 0 ? 0 : 1 + rng() % (rep % 4 == 0 ? 3000000 : 20000);
      segs.push_back(Seg{addr, addr + (1ull << 40), off, n});
      addr += (n * tes + 255) / 256 * 256 + 256;
      off += (n * bes + 15) / 16 * 16;
    }
    check(segs, chunk_units, tes, bes);
  }
  // sizes around the group boundaries
  for (uint64_t chunks : {1ull, 31ull, 32ull, 33ull, 511ull, 512ull, 513ull, 4096ull, 16384ull, 16385ull, 40000ull}) {
    std::vector<Seg> segs = {Seg{1 << 20, 1ull << 40, 0, chunks * 1024 - 3}};
    check(segs, 1024, 4, 4);
  }
  check({}, 1024, 4, 4);
  // the branch-free tile order of the contiguous kernels agrees with xcd_chunk
  for (uint64_t blocks : {1ull, 7ull, 512ull, 513ull, 2000ull, 15267ull, 40000ull, 300000ull}) {
    const XcdOrder o = xcd_order(blocks, 4096);
    const uint32_t run = xcd_run(blocks, 4096);
    for (uint64_t b = 0; b < blocks; b += (blocks > 5000 ? 7 : 1)) {
      const uint32_t mask = (8u << o.shift) - 1, w = (uint32_t)b & mask;
      const uint32_t permuted = (uint32_t)b - w + ((w & 7u) << o.shift) + (w >> 3);
      const uint32_t tile = b < o.ordered ? permuted : (uint32_t)b;
      REQUIRE(tile == xcd_chunk(b, blocks, run));
    }
  }
  std::printf("table layout ok\n");
  return 0;
}
