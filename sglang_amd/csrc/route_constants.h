// Every measured constant of the dispatcher's time models, in one place.
//
// choose_route (gemm_w8a8.hip) and dma3_plan (gemm_fp8_dma3.hip) pick a kernel, a tile and a K split by comparing
// modelled times.  The models' coefficients were fitted to timings on MI355X; they are data, not logic, so they live in
// this table, each with the measurement it comes from (the rocprofv3 summaries of the same shapes are under profiles/).
// Run-to-run and box-to-box spread of these timings is +-3 %; tests/test_gemm_routes_cpu.py perturbs every entry by
// +-10 % through mi355_gemm_plan_perturbed and holds the benchmark shapes on their kernels, or names the measured times
// of both candidates where a shape sits on a boundary.
#pragma once

namespace mi355 {

struct RouteConstants {
  // ---- two-phase 256 x 256 kernels (gemm_fp8_pp.hip, gemm_int8_pp.hip): a round of tiles takes
  //      (K blocks) * us_per_kblock + us_per_tile, whatever part of the tile is filled and however many CUs the round uses.
  //      K sweep at M = 4096, N = 36864 (K = 128 ... 14336): slope and intercept of the tile time.
  double pp_fp8_us_per_kblock = 1.39;
  double pp_int8_us_per_kblock = 1.46;  // K = 4096 -> N = 28672 at M = 4096: 32 K blocks in 57 us per round
  double pp_us_per_tile = 11.0;         // launch to first MFMA 2.7 + convert and stage 2.4 + output burst 5 + rest
  // ---- three-stage kernels with 64- or 128-token tiles (gemm_fp8_dma3.hip, gemm_int8_dma3.hip).  Per K block a
  //      workgroup takes the largest of: its tile's own time, a latency floor while its weight rows stream from HBM, its
  //      share of the chip's streaming rate.  Fitted to a sweep of 24 shapes x every (tile, split) (FP8) and to
  //      K = 4096 -> N = 4096 ... 28672, K = 14336 -> N = 4096 at 24 ... 1024 tokens (INT8).
  double dma3_hbm_bytes_per_us = 5.5e6;  // streaming rate of the 8-rows x 128-B access shape with two blocks in flight per CU
  // order: 128x256, 64x256, 128x128, 64x128, 128x192, 64x192 (token x channel tile); [0] FP8, [1] INT8 (no 192-wide tiles).
  // The INT8 128x256 entry is the two-phase 128-token kernel (gemm_int8_pp128.hip), 0.84 us; the lockstep kernel it
  // replaced took 1.14 us (M=4096 K=4096 N=1536: 42.0 -> 30.8 us, M=1024 N=6144: 42.1 -> 30.6, M=256 N=28672: 55.8 -> 44.6).
  double dma3_tile_us[2][6] = {{0.88, 0.58, 0.52, 0.40, 0.68, 0.50}, {0.84, 0.71, 0.64, 0.44, 0.0, 0.0}};
  double dma3_latency_us[2][6] = {{1.2, 1.0, 0.7, 0.51, 1.0, 0.75}, {0.96, 0.68, 0.59, 0.54, 0.0, 0.0}};
  double dma3_busy_chip_factor = 1.2;    // on the tile's own time in a round that keeps > 200 CUs multiplying: the clock drops
  double dma3_long_row_factor = 1.2;     // on the latency floor for weight rows longer than 8 KB (K = 18432 against K = 7168)
  double dma3_split_fixed_us = 8.0;      // a K split costs its fp32 partial traffic plus fixed + per_split * splits us
  double dma3_split_per_split_us = 0.25; //   (reduce launch and its pass over the partial tiles)
  double dma3_min_efficiency = 0.30;     // below this byte-model score of its best tiling (no split possible: N % 4 != 0)
                                         //   the generic kernel does better
  double dma3_small_tile_factor = 0.65;  // the byte-model score of 64-token tiles above 128 tokens
  // ---- decode sizes (M <= 16): the kernel that splits K over the waves of a workgroup (gemm_decode_wavesplit.hip) against
  //      the streaming kernel with its reduce launch (gemm_fp8_decode.hip).  Median launch, us, wave-split / streaming:
  //      FP8  7168->36864: M=1 48.1/52.1, 2 50.3/53.0, 3 51.8/53.9, 4 54.3/54.3, 8 62.7/56.9, 16 74.2/59.8;
  //      18432->7168: M=1 27.2/30.6, 2 28.0/31.3, 4 30.1/31.5, 8 33.5/32.1, 16 38.4/33.3;  7168->2048: M=2 9.3/10.9, 4 9.6/11.1,
  //      8 10.4/11.1, 16 11.7/10.9 (128 workgroups: half the CUs);  7168->4096: M=2 9.5/12.1, 16 11.6/12.6;  2048->7168: M=2
  //      8.7/11.0, 16 9.0/11.2;  M=4: 7168->1536 9.8/11.0, 1536->24576 12.2/13.4, 512->32768 14.6/8.9.
  //      INT8 M=1: 4096->6144 10.2/11.4, 4096->28672 24.7/30.9, 14336->4096 14.5/18.4;  M=16: 4096->6144 12.4/12.1,
  //      4096->28672 33.0/35.1, 14336->4096 18.2/19.7.
  //      Every token row costs the wave-split kernel a pass over K from L2 per workgroup, so it wins for few tokens or small
  //      weights; the INT8 streaming kernel is slower than the FP8 one, so there it wins at every decode size.
  double wavesplit_min_kblocks = 8.0;              // shorter K: one block per wave, the streaming kernel's wide tiles win
  double wavesplit_small_weight_bytes = 32e6;      // FP8: up to here the second launch it saves outweighs the token traffic ...
  double wavesplit_small_weight_max_tokens = 8.0;  // ... for this many tokens, or for any M <= 16 once N / 16 fills the CUs
  double wavesplit_large_weight_max_tokens = 4.0;  // FP8, larger weights: the token traffic decides
};
constexpr int ROUTE_CONSTANT_COUNT = sizeof(RouteConstants) / sizeof(double);
static_assert(sizeof(RouteConstants) == ROUTE_CONSTANT_COUNT * sizeof(double), "the table is read as an array of doubles");

// The table the calling thread's dispatcher uses: the defaults above, or the perturbed copy a plan query installed.
const RouteConstants& route_constants();
const char* route_constant_name(int index);

}  // namespace mi355
