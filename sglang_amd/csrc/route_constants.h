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
  double wavesplit_large_weight_max_tokens = 4.0;  // FP8, larger weights, one channel tile per workgroup: the token traffic decides
  // ---- two channel tiles (32 channels) per workgroup: a block's token fragment serves both, so the tokens' share of the
  //      L2 traffic halves, at half the workgroups.  FP8, median launch, us, one tile / two tiles / streaming kernel:
  //      7168->36864: M=1 48.0/50.2/51.5, 2 49.8/50.8/53.0, 3 52.0/51.4/54.0, 4 54.3/52.2/54.4, 8 62.6/54.3/57.1, 12 69.7/57.8/58.1,
  //      16 74.0/61.5/60.3;  18432->7168: M=1 27.2/25.9/30.5, 4 29.8/26.2/31.5, 8 33.2/27.3/32.1, 16 38.3/30.0/33.4;  1536->24576:
  //      M=1 11.3/11.0, 8 13.2/11.8/13.6;  7168->8192: M=1 14.5/14.7, 3 15.0/14.8, 8 17.0/15.2/17.7;  4096->14336: M=1 15.6/15.2,
  //      8 17.6/16.0/19.6;  7168->4096 (128 workgroups of two tiles): M=4 9.8/13.3, 16 11.7/15.3;  7168->2048: 9.8/13.3.
  //      INT8 stays on one tile: 4096->28672 M=4 25.4/29.1, 8 27.4/29.6, 16 32.8/31.0; 14336->4096 M=4 14.8/21.3; 4096->6144 10.7/10.4.
  double wavesplit_two_tile_min_workgroups = 200.0;  // N / 32 from here on
  double wavesplit_two_tile_min_tokens = 3.0;        // ... and from this many tokens on,
  double wavesplit_two_tile_long_k_blocks = 64.0;    // ... or at any token count once K has more blocks than this (four-wave workgroups)
  double wavesplit_two_tile_max_tokens = 12.0;       // FP8, larger weights, two tiles: up to here against the streaming kernel,
  double wavesplit_long_k_max_tokens = 16.0;         // ... and up to here beyond wavesplit_two_tile_long_k_blocks
  // ---- the mid-M kernel at decode sizes (FP8, 4 .. 16 tokens padded to one 64-token tile, K unsplit): where unsplit tiles fill
  //      most of the CUs in one round it streams the weight in one launch with 8-row x 128-byte loads.  Median launch, us,
  //      mid-M kernel (token scales M-major with an aligned pitch; 3.5-4 us more when they have to be re-laid out first) /
  //      streaming kernel + reduce at M = 16: 7168->36864 50.1 / 59.9, 7168->24576 36.4 / 43.2, 4096->28672 30.5 / 34.2,
  //      2048->32768 16.6 / 20.2, 1536->24576 10.7 / 14.3; 7168->18432 (144 workgroups) 33.3 / 33.9; and where the streaming
  //      kernel needs no split: 1024->65536 17.9 / 16.9, 512->32768 9.0 / 9.0.  Against the wave-split kernel (two tiles) at
  //      M = 4 / 8 / 12: 7168->36864 (192-channel tiles) 49.6 / 49.9 / 50.2 against 52.0 / 54.6 / 57.7; with 128-channel tiles
  //      7168->24576 35.8 / 36.0 / 36.2 against 34.3 / 36.1 / 38.3, 4096->28672 30.5 against 27.1 at M = 6, 2048->32768 16.6
  //      against 14.8: so only the 192-channel tiling replaces the wave-split kernel.
  double decode_dma3_min_tokens = 4.0;        // below, its token-scale quads do not exist and the wave-split kernel is as fast
  double decode_dma3_wavesplit_min_kblocks = 44.0;  // ... and replaces the wave-split kernel only for K of more blocks than this
                                                    // (M = 8: 7168->33280 47.2 against 53.6, 7168->49152 62.5 against 66.4, but
                                                    // 4096->33280 36.0 against 31.4: one turn of the wave-split ring covers K = 4096)
  // INT8 (the wave-split kernel has one channel tile per workgroup there, so its time grows faster with the tokens), median
  // launch, us, wave-split / mid-M kernel at M = 4 / 8 / 16: 7168->24576 37.6 / 42.2 / 50.5 against 37.9 / 37.6 / 38.3,
  // 2048->32768 16.2 / 18.1 / 21.1 against 17.4 / 17.4 / 17.8, 7168->36864 (144 tiles of 256 channels) 54.3 / 61.8 / 74.6
  // against 58.3 / 58.5 / 59.6, 4096->28672 25.5 / 27.3 / 33.0 against 31.9 / 31.9 / 32.1
  // (with six stages for the 64 x 128 tile: 7168->24576 35.5 / 35.6 / 36.2, 7168->36864 58.5 / 58.6 / 59.5, 4096->28672 31.2 / 31.1 / 31.4)
  double decode_dma3_int8_long_k_min_tokens = 8.0;  // ... from here on where K has more blocks than decode_dma3_wavesplit_min_kblocks,
  double decode_dma3_int8_min_tokens = 12.0;        // ... from here on for any K
  double decode_dma3_int8_min_workgroups = 130.0;
  double decode_dma3_min_workgroups = 170.0;  // unsplit tiles (of the channel width that gives most), at most one per CU: 192 and more measured, 144 not enough
  // ---- one-call linear at decode sizes.  Where the GEMM's plan is the mid-M kernel (above), that kernel's producer waves
  //      quantize the tokens: fused / quantizer launch + GEMM, us: 7168->36864 M=8 50.7 / 53.6, 16 51.5 / 54.0; 1536->24576 M=16
  //      13.7 / 15.1; 4096->28672 33.6 / 35.0; 1152->53248 17.8 / 20.7.  Otherwise:
  //      the streaming kernel with the quantizer in its prologue (one launch) against a
  //      quantizer launch + the wave-split kernel, where that is the GEMM's plan.  FP8, median call, us, fused / two launches:
  //      7168->36864: M=1 52.0/52.3, 4 54.6/56.2, 8 58.3/58.6;  18432->7168: M=1 30.8/30.1, 4 32.1/30.4, 8 33.6/31.6, 16 36.6/34.8;
  //      1536->24576: M=1 13.5/15.5, 4 14.0/15.7, 8 15.1/16.3;  7168->4096: M=1 11.9/13.7, 8 13.5/14.5, 16 16.0/15.9;
  //      7168->2048: M=1 10.3/13.2, 8 12.2/14.5;  2048->7168: M=1 10.5/11.5, 4 10.9/11.9, 8 12.2/12.0, 16 14.4/11.8.
  //      Beyond the GEMM's own plan the producer-wave kernel also takes the linear for fewer tokens on the same shapes
  //      (7168->36864 M=1 / 2 / 3: 50.2 / 50.2 / 50.3 against 52.0 / 53.4 / 54.7 on the fused streaming kernel) and where the
  //      streaming kernel would cut K into many ranges (7168->24576, seven: M=1 / 8 / 12 36.5 / 37.2 / 37.8 against 37.9 / 42.3 /
  //      44.4; not 4096->28672, four: M=1 32.3 against 29.6; two ranges: 1536->24576 13.1 against 13.5, 2048->32768 18.3 / 18.9)
  double linear_producer_min_decode_splits = 5.0;
  double fused_quant_long_k_blocks = 64.0;       // beyond this many K blocks the two launches win
  double fused_quant_short_k_blocks = 16.0;      // up to this many K blocks they win too,
  double fused_quant_short_k_max_tokens = 8.0;   // ... above this many tokens
};
constexpr int ROUTE_CONSTANT_COUNT = sizeof(RouteConstants) / sizeof(double);
static_assert(sizeof(RouteConstants) == ROUTE_CONSTANT_COUNT * sizeof(double), "the table is read as an array of doubles");

// The table the calling thread's dispatcher uses: the defaults above, or the perturbed copy a plan query installed.
const RouteConstants& route_constants();
const char* route_constant_name(int index);

}  // namespace mi355
