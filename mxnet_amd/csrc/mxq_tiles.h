// Tile choice shared by the FC and the implicit-GEMM convolution launchers.
#ifndef MXQ_TILES_H_
#define MXQ_TILES_H_

namespace mxq {

enum class Tile {
  kL8,      // 256 x 256, 64-byte stages, 4-stage ring, pinned pipeline
  kW128x2,  // 256 x 128, 64-byte stages, 2-stage ring
  kW128K2,  // 256 x 128, 128-byte stages, 2-stage ring
  kM128x2,  // 128 x 128, 64-byte stages, 2-stage ring
  kM128K2,  // 128 x 128, 128-byte stages, 2-stage ring
  kS64x2,   // 64 x 64, 64-byte stages, 2-stage ring
  kS64x4,   // 64 x 64, 64-byte stages, 4-stage ring, pinned pipeline
  kS64K2    // 64 x 64, 128-byte stages, 2-stage ring
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
//    once it fills the chip, else 64 x 64 keeps every CU busy.
inline Tile choose_tile(long M, long N, long K, long cus) {
  auto tiles = [&](long bm, long bn) { return ((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
  if (K > 256 && N > 128 && 16 * tiles(256, 256) >= 9 * cus) return Tile::kL8;
  if (N <= 64) return (K >= 4096) ? Tile::kS64x4 : Tile::kS64x2;
  if (4 * tiles(256, 128) >= 3 * cus) return (K >= 512) ? Tile::kW128K2 : Tile::kW128x2;
  if (tiles(128, 128) >= cus) return (K >= 256) ? Tile::kM128K2 : Tile::kM128x2;
  return (K >= 512) ? Tile::kS64K2 : Tile::kS64x2;
}

}  // namespace mxq
#endif  // MXQ_TILES_H_
