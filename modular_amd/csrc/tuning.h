// Tuning switches of the kernel selection, read from the environment ONCE per process (at the first
// matmul) and kept as an immutable snapshot: no launch path calls getenv.  Tuning runs and tests that
// flip a switch between calls re-read the environment through maxfp8_tuning_reload().
//
//   MAXFP8_TILE=1..4           force a tile shape of the tiled matmul (grouped: 2 = 256-row tiles in one
//                              launch, 3 = no small tiles, 4 = no large-tile launch)
//   MAXFP8_SPLITK=n            force the K split of the tiled matmul
//   MAXFP8_ONE_REGION=1        never cut a matmul into two regions
//   MAXFP8_PERSIST=0           per-tile kernels instead of the persistent one
//   MAXFP8_W4=0 / 4 / 5 / 6    whole-tile matmuls: the four-wave kernel never / in 128 x 256 / 160 x 256 / 192 x 256 tiles
//   MAXFP8_W4_SPLIT=0 / 1      its last round of tiles cut into pieces along K: never / wherever a shape has a cut
//                              (default: where the cost model says it pays)
//   MAXFP8_STREAMK=0 / 2       never / always split the work of whole-tile matmuls evenly over the blocks
//                              (default 1: where the cost model says it pays)
//   MAXFP8_BIG_ROWS=n          grouped: slots with at least n rows use the large-tile launch (1024)
//   MAXFP8_GROUPED_PERSIST=0   grouped: two launches (large tiles / the rest) instead of the one persistent launch
//   MAXFP8_GROUPED_OVERLAP=0   grouped, two launches: in line on the caller's stream
//   MAXFP8_GROUPED_SHARE=x     grouped: scales the estimate of how much of the chip the small tiles need (0.5)
//   MAXFP8_SKINNY_ALDS=0       decode kernel: activations loaded per slab even where a wave's share of them fits LDS
//   MAXFP8_SKINNY=<ntw>4<KB>   force a shape of the weight-streaming kernel (e.g. 1408, 2416)
#pragma once

namespace maxfp8 {

struct Tuning {
  int tile = 0;
  int splitk = 0;
  bool one_region = false;
  bool persist = true;
  int w4 = -1;               // -1: the planner decides
  int w4_split = -1;         // the four-wave kernel's tail cut: -1 the planner decides, 0 never, 1 wherever the shape has one
  int streamk = 1;
  int big_rows = 1024;
  bool grouped_persist = true;
  bool grouped_overlap = true;
  float grouped_share = 0.5f;
  // The grouped matmul's full 192-row tiles on the four-wave kernel, beside the persistent launch of the rest (block
  // scaling; MAXFP8_GROUPED_W4 = 0: one persistent launch); the least number of rows for it (MAXFP8_GROUPED_W4_ROWS);
  // a factor on the other launch's estimated work when the blocks decide their shares (MAXFP8_GROUPED_W4_SHARE; a negative
  // value is the number of blocks that stay, outright: -160 keeps 160); which rows go to the four-wave launch beside the
  // full 192-row tiles (MAXFP8_GROUPED_W4_HOT_REST, MAXFP8_GROUPED_W4_COLD_ROWS: see w4_grouped_head_rows).
  bool grouped_w4 = true;
  int grouped_w4_rows = 4096;
  float grouped_w4_share = 0.6f;
  int grouped_w4_hot_rest = 32, grouped_w4_cold_rows = 128;
  int skinny = 0;
  bool skinny_alds = true;
  unsigned generation = 0;  // counts the reloads: part of the key of every cache that depends on the switches
};

const Tuning& tuning();
void tuning_reload();

}  // namespace maxfp8
