// Tile and K-split choice of the 8-bit GEMM (int8 / e4m3) for an aligned problem: the one place the
// decision lives (the launcher and the schedule query of the C ABI both call it).  Host code only.
#pragma once
#include <algorithm>

namespace tsr950 {

struct Gemm8Schedule {
  int tile_m;    // rows of the workgroup tile: 256 or 128 (tile kernel), 32 or 64 (few-row streaming kernel)
  int tile_n;    // columns: 256 (tile kernel) or 128 (streaming kernel's strip)
  int tile_k;    // bytes of K per step: 128 (tile kernel) or 64 (a streaming slice)
  int split_k;   // K slices summed by the split-sum kernel (1 = none; the streaming kernel always goes through it)
  bool skinny;   // the few-row streaming kernel
};

constexpr int kGemm8SkinnyMaxM = 64;

// Time estimate (microseconds) of `tiles` workgroup tiles of bm x 256 walking `ksteps` 128-deep K steps,
// fitted to timings of both tiles on this part over products from 1024^3 to 8192^3: rounds of 256
// concurrent tiles; a tile's cost outside its K loop grows with the number of tiles storing at once, and
// a K step is slower with every compute unit busy (the board's power limit sets the clock).
inline double est_tiles8_us(int bm, long tiles, int ksteps) {
  const double f0 = bm == 256 ? 9.6 : 6.0, f1 = 3.0, s0 = bm == 256 ? 1.2 : 0.62, s1 = bm == 256 ? 0.48 : 0.30;
  const long full = tiles / 256, rem = tiles % 256;
  double t = (double)full * (f0 + f1 + ksteps * (s0 + s1));
  if (rem) t += f0 + f1 * rem / 256.0 + ksteps * (s0 + s1 * std::min(1.0, std::max(0.0, (rem - 144) / 112.0)));
  return t;
}

inline Gemm8Schedule select_gemm8_schedule(int M, int N, int K) {
  auto cdiv = [](long a, long b) { return (a + b - 1) / b; };
  // At most 64 rows against a long K (quantised decode): the streaming kernel, one workgroup per
  // 128-column strip and K range, about one workgroup per compute unit and at least two 64-row
  // slices for each of its waves (8 waves up to 32 rows, 4 above: twice the accumulators).
  if (M <= kGemm8SkinnyMaxM && K % 64 == 0 && K >= 2048) {
    const int nw = M <= 32 ? 8 : 4;
    const int strips = (int)cdiv(N, 128);
    int splits = std::max(1, std::min((256 + strips / 2) / strips, K / (2 * nw * 64)));
    const int kps = (int)cdiv(cdiv(K, splits), 64) * 64;
    return {M <= 32 ? 32 : 64, 128, 64, (int)cdiv(K, kps), true};
  }
  // Tile rows (256 or 128) and K slices by estimated time.  Few tiles and a long K (few rows against a
  // big weight matrix): K is split over the idle compute units (a power of two, tiles x slices within
  // the 256 compute units, every slice at least 512 deep); the sum over the slices reads the partials
  // and writes the result at about 4.4 TB/s.
  const int ksteps = (int)cdiv(K, 128);
  const long tn = cdiv(N, 256);
  Gemm8Schedule best{256, 256, 128, 1, false};
  double best_us = 1e30;
  for (int cand : {256, 128}) {
    const long tiles = cdiv(M, cand) * tn;
    const double us1 = est_tiles8_us(cand, tiles, ksteps);
    if (us1 < best_us) { best_us = us1; best.tile_m = cand; best.split_k = 1; }
    if (tiles <= 128)
      for (int sp = 2; sp <= 16 && tiles * sp <= 256 && K / sp >= 512; sp *= 2) {
        const double us = est_tiles8_us(cand, tiles * sp, (int)cdiv(ksteps, sp)) + 2.0 +
                          (double)M * N * (4.0 * sp + 4.0) / 4.4e6;
        if (us < best_us) { best_us = us; best.tile_m = cand; best.split_k = sp; }
      }
  }
  return best;
}

}  // namespace tsr950
