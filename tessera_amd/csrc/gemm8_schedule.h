// Tile and K-split choice of the 8-bit GEMM (int8 / e4m3) for an aligned problem: the one place the
// decision lives (the launcher and the schedule query of the C ABI both call it).  Host code only.
#pragma once
#include <algorithm>
#include <cmath>

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

// Time estimate (microseconds) for up to 1024 rows against a weight matrix that streams from HBM,
// fitted (10 % rms) to 2300 timings of forced schedules on this part — the streaming kernel and the
// 128- and 256-row tiles, K in 1 to 32 parts, 18 weight shapes from 2048 x 7168 to 32768 x 4096 (the
// weights cycled through copies) under 16 to 1024 rows: a launch cost, then the larger of the busiest
// compute unit's K steps (its first workgroup at `step`, every further one sharing the unit at
// `shared` per step) and the time to stream the tile columns of B at `tbs` TB/s, which takes about
// 155 workgroups in flight to reach (256 for the streaming kernel) and is stretched by a last, partly filled round; the sum over
// K parts (always there behind the streaming kernel) adds 2 us and 1.4 us per million partials.
struct Gemm8Fit { double launch, step, shared, tbs; };
constexpr Gemm8Fit kGemm8Fit[3] = {{5.23, 0.731, 1.265, 5.44},     // the streaming kernel (a step = one 64-row slice of a wave)
                                   {6.51, 0.780, 1.121, 6.52},     // 128 x 256 tiles (a step = 128 of K)
                                   {9.82, 1.107, 1.944, 5.31}};    // 256 x 256 tiles
inline double est_gemm8_fit_us(int kind, int M, int N, int K, int splits) {
  const Gemm8Fit& f = kGemm8Fit[kind];
  const long cols = kind == 0 ? (N + 127) / 128 : (N + 255) / 256;
  const long rows = kind == 0 ? 1 : kind == 1 ? (M + 127) / 128 : (M + 255) / 256;
  const long wgs = rows * cols * splits;
  // (the streaming kernel's waves share a workgroup's K range: 8 waves of one 32-row block, or 4 of two)
  const double steps = kind == 0 ? (double)K / 64 / splits / (M <= 32 ? 8 : 2) : (double)K / 128 / splits;
  const double busiest = (double)((wgs + 255) / 256);
  const double compute = steps * (f.step + f.shared * (busiest - 1.0));
  const double bytes = (double)K * cols * (kind == 0 ? 128 : 256);
  // (the fit put the rate's saturation at 155 workgroups for all three; the streaming kernel, one
  // workgroup per compute unit, is set to 256: the fit's largest misses were its runs at 144 workgroups,
  // measured a third slower than estimated, and over the fit's shapes the choices at 16 and 32 rows come
  // out 5 % faster with it)
  const double sat = kind == 0 ? 256.0 : 155.0;
  const double stream = bytes / (f.tbs * 1e6 * std::min(1.0, wgs / sat)) * (wgs > 256 ? busiest * 256.0 / wgs : 1.0);
  const double sum = (splits > 1 || kind == 0) ? 2.06 + (double)M * N * splits * 1.43e-6 : 0.0;
  return f.launch + std::max(compute, stream) + sum;
}

// The rule: the streaming kernel for few rows, else tile rows and a power-of-two K split by est_tiles8_us.
inline Gemm8Schedule select_gemm8_rule(int M, int N, int K) {
  auto cdiv = [](long a, long b) { return (a + b - 1) / b; };
  // At most 64 rows against a long K (quantised decode): the streaming kernel, one workgroup per
  // 128-column strip and K range, about one workgroup per compute unit and at least two 64-row
  // slices for each of its waves (8 waves up to 32 rows, 4 above: twice the accumulators).
  if (M <= kGemm8SkinnyMaxM && K % 64 == 0 && K >= 2048) {
    const int nw = M <= 32 ? 8 : 4;
    const int strips = (int)cdiv(N, 128);
    // (never a little over one workgroup per compute unit: the second round would be nearly empty)
    int splits = std::max(1, std::min(256 / strips, K / (2 * nw * 64)));
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

// The schedule of an aligned 8-bit product: the rule above, unless — for 16 to 1024 rows under a weight
// matrix of the sizes the fit covers — the fitted estimate finds a schedule it expects to be at least
// a tenth faster than the rule's (the fit's own error is a tenth: smaller promises are noise).  Over the
// fit's shapes the rule alone is 5 % behind the best forced schedule at 128 to 1024 rows and 13 to 22 %
// at 16 to 64; with this step 1 to 8 %.
inline Gemm8Schedule select_gemm8_schedule(int M, int N, int K) {
  auto cdiv = [](long a, long b) { return (a + b - 1) / b; };
  const Gemm8Schedule rule = select_gemm8_rule(M, N, K);
  if (!(M >= 16 && M <= 1024 && N >= 2048 && K >= 1024)) return rule;
  const double rule_us = est_gemm8_fit_us(rule.skinny ? 0 : rule.tile_m == 128 ? 1 : 2, M, N, K, rule.split_k);
  Gemm8Schedule best = rule;
  double best_us = 0.9 * rule_us;
  for (int kind = (M <= kGemm8SkinnyMaxM && K % 64 == 0) ? 0 : 1; kind < 3; ++kind)
    for (int sp : {1, 2, 3, 4, 5, 6, 7, 8, 12, 16, 24, 32}) {
      if (kind == 0 ? K / sp < 1024 : (K / sp < 512 || sp > 16)) continue;
      // (up to 32 rows a tile has to beat the streaming kernel by another 5 %: below the 16 rows the fit
      // starts at, that kernel is the faster by more)
      const double us = est_gemm8_fit_us(kind, M, N, K, sp) * (kind != 0 && M <= 32 ? 1.05 : 1.0);
      if (us >= best_us) continue;
      best_us = us;
      if (kind == 0) {
        const int kps = (int)cdiv(cdiv(K, sp), 64) * 64;
        best = Gemm8Schedule{M <= 32 ? 32 : 64, 128, 64, (int)cdiv(K, kps), true};
      } else {
        best = Gemm8Schedule{kind == 1 ? 128 : 256, 256, 128, sp, false};
      }
    }
  return best;
}

}  // namespace tsr950
