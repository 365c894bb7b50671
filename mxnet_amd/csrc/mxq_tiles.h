// Tile choice shared by the FC and the implicit-GEMM convolution launchers.
#ifndef MXQ_TILES_H_
#define MXQ_TILES_H_

#include <cstddef>

namespace mxq {

// What a caller may pin instead of leaving it to the choosers below: a tile configuration
// number of the launcher (0 = choose by shape), the number of work-groups that share one
// output tile along K (0 = choose, 1 = no split) and, for the short-K streaming kernel,
// its work-groups per CU (0 = choose).  The operator entry points pass the default; the
// test-only entry points pass what the test asks for.
struct GemmForce {
  int cfg = 0;
  int splits = 0;
  int stream_groups = 0;
};

// Caller-provided scratch for the split-K route (may be null: then nothing is split).
struct Workspace {
  void* ptr = nullptr;
  size_t bytes = 0;
};

enum class Tile {
  kL8,      // 256 x 256, 64-byte stages, 4-stage ring, pinned pipeline
  kW128x2,  // 256 x 128, 64-byte stages, 2-stage ring
  kW128K2,  // 256 x 128, 128-byte stages, 2-stage ring
  kM128x2,  // 128 x 128, 64-byte stages, 2-stage ring
  kM128K2,  // 128 x 128, 128-byte stages, 2-stage ring
  kS64x2,   // 64 x 64, 64-byte stages, 2-stage ring
  kS64x4,   // 64 x 64, 64-byte stages, 4-stage ring, pinned pipeline
  kS64K2,   // 64 x 64, 128-byte stages, 2-stage ring
  kS64K4,   // 64 x 64, 256-byte stages, 2-stage ring
  kR128K2,  // 128 x 64, 128-byte stages, 2-stage ring
  kQ128K2,  // 64 x 128, 128-byte stages, 2-stage ring
  kW192K2   // 256 x 192, 128-byte stages, 2-stage ring
};

// M x N outputs, reduction length K, `cus` compute units.  Distilled from sweeps over
// BERT-, ResNet-50- and square shapes (each rule names the measurement behind it):
//  * the 256 x 256 tile wins from about 0.56 tiles per CU on (4096 x 2304 x 768: 144 tiles,
//    15.9 us against 20.4 us for 128 x 128), if the output is wider than 128 columns and K
//    is long enough to amortise its prologue and epilogue;
//  * outputs of at most 64 columns take the 64 x 64 tile (nothing wider is useful);
//  * otherwise the 2-stage rings win: they need little LDS, several work-groups share a
//    CU, and one group's epilogue overlaps another's K loop.  A K step costs a barrier and
//    a round of DMA latency whatever its size, so from K = 512 on the stages are 128 bytes
//    deep (half as many steps: 10-20 % on every mid-size shape measured); below that the
//    deeper stage would mostly be padding or leave too few steps to overlap;
//  * 256 x 128 from 0.75 tiles per CU (fewer, larger stores per loaded byte), 128 x 128
//    once it fills the chip, then 128 x 64 / 64 x 128, else 64 x 64 keeps every CU busy.
// `gather` says that the left operand is gathered pixel by pixel (convolution): the 64-row
// tile then issues half as many gathers per wave and measures a few per cent ahead of the
// 128-row one, which in turn is ahead for plain row-major operands.
inline Tile choose_tile(long M, long N, long K, long cus, bool gather = false,
                        int* splits = nullptr) {
  if (splits != nullptr) *splits = 1;
  auto tiles = [&](long bm, long bn) { return ((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
  // an output whose width is a multiple of 192 and that gives 256 x 192 tiles to (nearly)
  // every CU exactly once: 4096 x 768 -> 3072 is 256 such tiles against 192 of 256 x 256 on
  // 256 CUs (15.9 against 17.0 us), -> 2304 is 192 against 144 (15.4 against 16.1 us)
  if (!gather && K >= 512 && N % 192 == 0 && tiles(256, 192) <= cus &&
      4 * tiles(256, 192) >= 3 * cus && tiles(256, 192) > tiles(256, 256))
    return Tile::kW192K2;
  if (K > 256 && N > 128 && 16 * tiles(256, 256) >= 9 * cus) return Tile::kL8;
  // Split-K: an output of few 64 x 64 tiles under a very long reduction (a fully-connected
  // layer at small batch: 256 x 8192 -> 800, 64 x 25088 -> 4096) leaves most CUs idle and
  // each tile walks thousands of K bytes alone.  Up to four work-groups share a tile then
  // (18.3 -> 12.9 us and 63.5 -> 27 us on those two).  The price is a counter-clearing
  // launch and the partial sums' round trip through memory (about 2 us plus 1 us per 4 MB),
  // which is why shapes with more tiles or a shorter K are left alone: on the ResNet-50 and
  // BERT layers every split measured slower than the unsplit kernel.
  auto few_tile_splits = [&]() {
    const long t = tiles(64, 64);
    if (splits == nullptr || K < 8192 || 2 * t > cus) return;
    long sp = cus / t;
    if (sp > 4) sp = 4;
    if (sp >= 2) *splits = static_cast<int>(sp);
  };
  if (N <= 64) {
    if (K >= 4096) few_tile_splits();
    return (K >= 4096) ? Tile::kS64x4 : Tile::kS64x2;
  }
  if (4 * tiles(256, 128) >= 3 * cus) return (K >= 512) ? Tile::kW128K2 : Tile::kW128x2;
  if (tiles(128, 128) >= cus) return (K >= 256) ? Tile::kM128K2 : Tile::kM128x2;
  if (K < 512) return Tile::kS64x2;
  // half-size tiles while they still give every CU one: 12544 x 2304 -> 256 takes 14.1 us on
  // 392 tiles of 64 x 128 against 17.6 us on 784 tiles of 64 x 64.  From K = 4096 on the
  // 64 x 64 tile with 256-byte stages is the better of the two unless the half-size tiles
  // still come two to a CU (512 x 4096 -> 4096: 18.3 us against 19.8 us on 256 tiles).
  const long tq = tiles(64, 128), tr = tiles(128, 64);
  const long need = (K >= 4096) ? 2 * cus : cus;
  if (tq >= need || tr >= need) {
    const bool q_fits = tq >= need && N % 128 == 0, r_fits = tr >= need;
    if (q_fits && (gather || !r_fits)) return Tile::kQ128K2;
    return r_fits ? Tile::kR128K2 : Tile::kQ128K2;
  }
  // Fewer than two 64 x 64 tiles per CU are left: 256-byte stages once K leaves them four
  // steps (3136 x 4608 -> 512: 15.8 us against 19.8 us).  With so few work-groups per CU a
  // deeper stage is what keeps bytes in flight, which counts most when the operands come
  // from HBM: inside the 19-layer ResNet stack (every layer reads operands last touched
  // 300 us earlier) 3136 x 2048 -> 512 is 3.6 us and the strided 3136 x 1024 -> 512 2.4 us
  // faster this way, and level with 128-byte stages when the operands are cache-warm.
  if (K >= 4096) few_tile_splits();
  return (K >= 1024) ? Tile::kS64K4 : Tile::kS64K2;
}

}  // namespace mxq
#endif  // MXQ_TILES_H_
