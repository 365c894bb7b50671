// Tile choice shared by the FC and the implicit-GEMM convolution launchers.
#ifndef MXQ_TILES_H_
#define MXQ_TILES_H_

namespace mxq {

enum class Tile {
  kL8,      // 256 x 256, 4-stage ring, pinned pipeline
  kW128x2,  // 256 x 128, 2-stage ring
  kM128x2,  // 128 x 128, 2-stage ring
  kM128x4,  // 128 x 128, 4-stage ring, pinned pipeline
  kS64x2,   // 64 x 64, 2-stage ring
  kS64x4    // 64 x 64, 4-stage ring, pinned pipeline
};

// M x N outputs, reduction length K, `cus` compute units.  Distilled from sweeps over
// BERT-, ResNet-50- and square shapes (each rule names the measurement behind it):
//  * the 256 x 256 tile wins once it fills the chip, the output is wider than 128
//    columns and K is long enough to amortise its prologue and epilogue;
//  * outputs of at most 64 columns take the 64 x 64 tile (nothing wider is useful);
//  * otherwise the 2-stage rings win: they need a quarter of the LDS, several
//    work-groups share a CU, and one group's epilogue overlaps another's K loop.
//    Short K prefers the 256 x 128 tile (fewer, larger stores per loaded byte);
//  * long K (>= 2048) with about one 128 x 128 tile per CU is the one mid-size case
//    where the deeper ring pays, and with too few 128 x 128 tiles for the chip the
//    64 x 64 tile keeps every CU busy.
inline Tile choose_tile(long M, long N, long K, long cus) {
  auto tiles = [&](long bm, long bn) { return ((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
  if (K > 256 && N > 128 && tiles(256, 256) >= cus) return Tile::kL8;
  if (N <= 64) return (K >= 4096) ? Tile::kS64x4 : Tile::kS64x2;
  const long t128 = tiles(128, 128);
  if (K <= 512 && tiles(256, 128) >= cus) return Tile::kW128x2;
  if (t128 >= cus) return (K >= 2048) ? Tile::kM128x4 : Tile::kM128x2;
  if (K >= 2048 && 4 * t128 >= 3 * cus) return Tile::kM128x4;
  return (K >= 4096) ? Tile::kS64x4 : Tile::kS64x2;
}

}  // namespace mxq
#endif  // MXQ_TILES_H_
