// Decode (M <= 16) GEMMs for gfx950 when the weight is small - blockwise-scaled FP8 and per-token x per-channel INT8:
// K is split over the WAVES of a workgroup, and the sum is finished inside the workgroup.
//
// The streaming decode kernel (gemm_fp8_decode.hip) gives a workgroup 128 channels and 8 K blocks; a weight of a few MB
// (K = 7168 -> N = 2048: 14 MB) then makes ~100 workgroups, half the CUs stay empty, and a second launch adds the K
// ranges.  Both cost more than the traffic itself: 6.1 us + 2.8 us for a weight that leaves HBM in 2 us.  Here a workgroup
// owns 16 channels - one MFMA tile for the <= 16 tokens - over ALL of K; its W waves take K blocks w, w + W, w + 2 W, ...
// so that neighbouring waves read neighbouring 128-byte pieces of the same weight rows.  A wave requests its blocks
// straight into registers in MFMA operand layout (two 16-byte pieces per lane and block for the weight, two for the
// tokens, which come from L2 after the first workgroups touched them), multiplies them as they arrive, and the W partial
// tiles are added through LDS in wave order by wave 0, which applies the epilogue and stores.
// No workspace, no second launch, N / 16 workgroups - or N / 32 with two channel tiles each (FP8, where wavesplit_two_tiles
// says so): a block's token fragment then serves both tiles, which halves what the tokens add to a workgroup's L2 traffic.
//
// A wave keeps a ring of KBW register slots: a slot is multiplied and requested again at once for the block KBW further
// on, so KBW - 1 blocks stay in flight for as long as K lasts (requesting KBW blocks together and waiting for all of
// them left nothing in flight between such rounds: K = 18432 -> N = 7168 at M = 1 30.4 -> 27.2 us, INT8 K = 14336 -> N = 4096
// 15.6 -> 14.5 us; shapes of one or two turns are unchanged).  ~80-90 registers: five waves per SIMD (two tiles: 118-128, four waves).
// Blocks past the end of K are fetched from the last valid block and multiply a zero scale (FP8) or zeroed tokens (INT8).
// Requires K % 128 == 0, N % 16 == 0, 16-byte aligned rows.  FP8 sums differ from the streaming kernel's in the order of
// the additions only (per wave in K order, then over waves); INT8 results are exact either way.
#include "gemm_common.h"

namespace mi355 {
namespace {

typedef const __attribute__((address_space(4))) float* cfloat_ptr;

struct Frag {
  u32x4 lo, hi;
};
__device__ __forceinline__ v8i as_v8i(const Frag& f) {
  return v8i{(int)f.lo.x, (int)f.lo.y, (int)f.lo.z, (int)f.lo.w, (int)f.hi.x, (int)f.hi.y, (int)f.hi.z, (int)f.hi.w};
}

// UE8M0 (FP8 only): p.sa / p.sb point to 32-bit words of four exponent bytes (token words M-major: word (kb >> 2) * sa_sk + m;
// weight words one row per weight row: (kb >> 2) * sb_sk + n * sb_sn, constant over a 128-row block) and the MFMA applies
// them itself (v_mfma_scale_f32_16x16x128_f8f6f4: the weight row's byte with the A operand, the token's with the B
// operand), accumulating in place: no scale arithmetic, no expansion of the exponents to fp32 in front of the GEMM.
// CT: MFMA channel tiles per workgroup (16 or 32 channels).  With two, a block's token fragment is fetched once for both:
// the tokens' share of what a workgroup pulls from L2 halves, which matters from about five tokens on.
template <bool IS_FP8, int W, int KBW, bool UE8M0 = false, int CT = 1>
__global__ __launch_bounds__(64 * W) __attribute__((amdgpu_waves_per_eu(CT == 2 ? 4 : 5))) void decode_wavesplit_kernel(const GemmParams p) {
  static_assert(IS_FP8 || !UE8M0, "exponent scales belong to the FP8 path");
  static_assert(CT == 1 || CT == 2, "one or two channel tiles");
  using AccT = typename std::conditional<IS_FP8, float, int>::type;
  typedef AccT acc4 __attribute__((ext_vector_type(4)));
  __shared__ acc4 red[W][CT][64];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l16 = lane & 15, q = lane >> 4;
  const int n0 = blockIdx.x * (16 * CT);  // (a multiple of 32 for CT = 2: both tiles lie in one 128-channel scale block)
  const int tok = min(l16, p.M - 1);  // lanes past M repeat the last token; their results are never stored
  // operand layout of the 16 x 16 x 128 MFMA: lane (row l16, quarter q) holds bytes [16 q, +16) and [64 + 16 q, +16) of the row's block
  const uint8_t* wrow = p.b + (int64_t)(n0 + l16) * p.ldb + q * 16;
  const uint8_t* trow = p.a + (int64_t)tok * p.lda + q * 16;
  const float* sa_row = IS_FP8 ? p.sa + (int64_t)tok * p.sa_sm : nullptr;
  // wave-uniform, read through the constant address space: scalar loads, which the vector-memory counter does not see
  const cfloat_ptr sb_row = (cfloat_ptr)(IS_FP8 ? p.sb + (int64_t)(UE8M0 ? n0 : (n0 >> 7)) * p.sb_sn : nullptr);

  acc4 acc[CT];
#pragma unroll
  for (int c = 0; c < CT; ++c) acc[c] = acc4{0, 0, 0, 0};
  // A ring of KBW register slots: the wave's i-th block is K block i * W + wave; slot j is multiplied and at once requested
  // again for the block KBW further on, so KBW - 1 blocks are always in flight (rounds of KBW blocks that are requested
  // together and awaited together leave the wave with nothing in flight between rounds).  Blocks past the end of K (the padding of the
  // last turn) clamp to the last one and contribute zero.
  // The loads and their waits are written as instructions: left to the compiler, the wait at the loop's back edge becomes
  // "everything but the newest block" and the ring runs empty once per turn.  A slot's registers are outputs of its request
  // and in-out operands of its wait, so no compiler-generated instruction touches them in between; vector loads complete in
  // order, so "at most (KBW - 1) blocks' loads outstanding" means the oldest slot has landed.
  constexpr int LOADS = 2 * CT + 2 + (IS_FP8 ? 1 : 0);  // per block: the halves of the weight and token fragments, the token scale (word)
  Frag wf[KBW][CT], tf[KBW];
  float sav[KBW], sbv[KBW];
  auto request = [&](int j, int i) {
    const int kc = min(i * W + wave, p.kb_total - 1);  // wave-uniform
    const uint8_t* wp = wrow + (int64_t)kc * KSTEP;
    const uint8_t* tp = trow + (int64_t)kc * KSTEP;
    asm volatile(
        "global_load_dwordx4 %0, %4, off\n\tglobal_load_dwordx4 %1, %4, off offset:64\n\t"
        "global_load_dwordx4 %2, %5, off\n\tglobal_load_dwordx4 %3, %5, off offset:64"
        : "=&v"(wf[j][0].lo), "=&v"(wf[j][0].hi), "=&v"(tf[j].lo), "=&v"(tf[j].hi)
        : "v"(wp), "v"(tp)
        : "memory");
    if constexpr (CT == 2) {
      const uint8_t* wp1 = wp + 16 * p.ldb;  // the same block of the next sixteen weight rows
      asm volatile("global_load_dwordx4 %0, %2, off\n\tglobal_load_dwordx4 %1, %2, off offset:64"
                   : "=&v"(wf[j][1].lo), "=&v"(wf[j][1].hi)
                   : "v"(wp1)
                   : "memory");
    }
    if constexpr (IS_FP8) {
      // fp32 scales: block kc's; packed exponents: the word that holds block kc's byte, kept as raw bits
      const float* sp = sa_row + (int64_t)(UE8M0 ? (kc >> 2) : kc) * p.sa_sk;
      asm volatile("global_load_dword %0, %1, off" : "=&v"(sav[j]) : "v"(sp) : "memory");
      sbv[j] = sb_row[(int64_t)(UE8M0 ? (kc >> 2) : kc) * p.sb_sk];  // wave-uniform: a scalar load, not counted in vmcnt
    }
  };
  // waits until at most `behind` blocks requested after slot j's are still outstanding: slot j has landed
  auto await = [&](int j, int behind) {  // `behind` is a constant at every call; the switch folds away
#define MI355_WS_AWAIT(NBLK)                                                                                                     \
  if constexpr (IS_FP8 && CT == 2)                                                                                               \
    asm volatile("s_waitcnt vmcnt(%7)" : "+v"(wf[j][0].lo), "+v"(wf[j][0].hi), "+v"(wf[j][1].lo), "+v"(wf[j][1].hi), "+v"(tf[j].lo), "+v"(tf[j].hi), "+v"(sav[j]) : "n"((NBLK)*LOADS)); \
  else if constexpr (IS_FP8)                                                                                                     \
    asm volatile("s_waitcnt vmcnt(%5)" : "+v"(wf[j][0].lo), "+v"(wf[j][0].hi), "+v"(tf[j].lo), "+v"(tf[j].hi), "+v"(sav[j]) : "n"((NBLK)*LOADS)); \
  else if constexpr (CT == 2)                                                                                                    \
    asm volatile("s_waitcnt vmcnt(%6)" : "+v"(wf[j][0].lo), "+v"(wf[j][0].hi), "+v"(wf[j][1].lo), "+v"(wf[j][1].hi), "+v"(tf[j].lo), "+v"(tf[j].hi) : "n"((NBLK)*LOADS)); \
  else                                                                                                                           \
    asm volatile("s_waitcnt vmcnt(%4)" : "+v"(wf[j][0].lo), "+v"(wf[j][0].hi), "+v"(tf[j].lo), "+v"(tf[j].hi) : "n"((NBLK)*LOADS))
    switch (behind) {
      case 3: MI355_WS_AWAIT(3); break;
      case 2: MI355_WS_AWAIT(2); break;
      case 1: MI355_WS_AWAIT(1); break;
      default: MI355_WS_AWAIT(0); break;
    }
#undef MI355_WS_AWAIT
  };
  auto multiply = [&](int j, int i) {
    const int kb = i * W + wave;
    const bool valid = kb < p.kb_total;
    if constexpr (UE8M0) {
      const int shift = 8 * (min(kb, p.kb_total - 1) & 3);
      const int ea = in_vgpr((int)((__float_as_uint(sbv[j]) >> shift) & 0xffu)), eb = (int)((__float_as_uint(sav[j]) >> shift) & 0xffu);
      const u32x4 z = {0u, 0u, 0u, 0u};
      Frag t = tf[j];
      if (!valid) t.lo = z, t.hi = z;  // a block past the end of K multiplies zeros
#pragma unroll
      for (int c = 0; c < CT; ++c)
        acc[c] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(as_v8i(wf[j][c]), as_v8i(t), acc[c], 0, 0, 0, ea, 0, eb);
    } else if constexpr (IS_FP8) {
      const float sc = valid ? sav[j] * sbv[j] : 0.f;
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        const v4f part = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(as_v8i(wf[j][c]), as_v8i(tf[j]), v4f{0.f, 0.f, 0.f, 0.f}, 0,
                                                                          0, 0, 0, 0, 0);
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[c][v] = fmaf(part[v], sc, acc[c][v]);
      }
    } else {
      const u32x4 z = {0u, 0u, 0u, 0u};
      const u32x4 tlo = valid ? tf[j].lo : z, thi = valid ? tf[j].hi : z;
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        const Frag& f = wf[j][c];
        acc[c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{(int)f.lo.x, (int)f.lo.y, (int)f.lo.z, (int)f.lo.w},
                                                       v4i{(int)tlo.x, (int)tlo.y, (int)tlo.z, (int)tlo.w}, acc[c], 0, 0, 0);
        acc[c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{(int)f.hi.x, (int)f.hi.y, (int)f.hi.z, (int)f.hi.w},
                                                       v4i{(int)thi.x, (int)thi.y, (int)thi.z, (int)thi.w}, acc[c], 0, 0, 0);
      }
    }
  };
  const int blocks = (p.kb_total + W * KBW - 1) / (W * KBW) * KBW;  // per wave, padded to whole turns of the ring
#pragma unroll
  for (int j = 0; j < KBW; ++j) request(j, j);
  // the fences keep the order "await and multiply slot j, request it again"
  int i0 = 0;
  for (; i0 + KBW < blocks; i0 += KBW) {
#pragma unroll
    for (int j = 0; j < KBW; ++j) {
      __builtin_amdgcn_sched_barrier(0);
      await(j, KBW - 1);
      multiply(j, i0 + j);
      __builtin_amdgcn_sched_barrier(0);
      request(j, i0 + j + KBW);
    }
  }
  // last turn: nothing is requested any more, so slot j has KBW - 1 - j blocks behind it
  static_assert(KBW == 4, "the last turn is written out for four slots");
  __builtin_amdgcn_sched_barrier(0);
  await(0, 3);
  multiply(0, i0);
  __builtin_amdgcn_sched_barrier(0);
  await(1, 2);
  multiply(1, i0 + 1);
  __builtin_amdgcn_sched_barrier(0);
  await(2, 1);
  multiply(2, i0 + 2);
  __builtin_amdgcn_sched_barrier(0);
  await(3, 0);
  multiply(3, i0 + 3);
  __builtin_amdgcn_sched_barrier(0);

  // ---- add the W partial tiles in wave order
  if (wave != 0) {
#pragma unroll
    for (int c = 0; c < CT; ++c) red[wave][c][lane] = acc[c];
  }
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int w = 1; w < W; ++w) {
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      const acc4 t = red[w][c][lane];
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[c][v] += t[v];
    }
  }
  if (l16 >= p.M) return;
  const bool vec_ok = ((p.ldo & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    // lane holds channels n .. n + 3 for token l16
    const int n = n0 + 16 * c + 4 * q;
    if constexpr (IS_FP8) {
      float r4[4] = {acc[c][0], acc[c][1], acc[c][2], acc[c][3]};
      fp8_channel_epilogue(p, n, r4);
      store_out4(p.out, p.out_dtype, (int64_t)l16 * p.ldo + n, r4, 4, vec_ok);
    } else if (p.out_dtype == MI355_I32) {
      int* o = reinterpret_cast<int*>(p.out) + (int64_t)l16 * p.ldo + n;
#pragma unroll
      for (int v = 0; v < 4; ++v) o[v] = acc[c][v];
    } else {
      const float sa_m = p.sa[l16];
      float r4[4];
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        // separately rounded multiply and add: the contract is mul, mul, add, not a fused multiply-add
        float t = mul_rn((float)acc[c][v], mul_rn(p.sb[n + v], sa_m));
        if (p.bias) {
          const uint32_t hb = reinterpret_cast<const uint16_t*>(p.bias)[n + v];
          t = add_rn(t, (p.out_dtype == MI355_BF16) ? bf16_bits_to_f32(hb) : f16_bits_to_f32(hb));
        }
        r4[v] = t;
      }
      store_out4(p.out, p.out_dtype, (int64_t)l16 * p.ldo + n, r4, 4, vec_ok);
    }
  }
}

template <bool IS_FP8, int W, int KBW, bool UE8M0 = false, int CT = 1>
int launch_variant(const GemmParams& p, hipStream_t stream, const char* what) {
  hipLaunchKernelGGL((decode_wavesplit_kernel<IS_FP8, W, KBW, UE8M0, CT>), dim3((unsigned)(p.N / (16 * CT))), dim3(64 * W), 0, stream, p);
  return check_launch(what);
}

template <bool IS_FP8, bool UE8M0 = false>
int launch_wavesplit(GemmParams& p, hipStream_t stream, const char* what) {
  p.splits = 1;
  p.tiles_m = 1;
  p.tiles_n = p.N / 16;
  const WavesplitShape s = wavesplit_shape(p.K);
  if (wavesplit_two_tiles(IS_FP8, p.M, p.N, p.K))
    return s.waves == 4 ? launch_variant<IS_FP8, 4, 4, UE8M0, 2>(p, stream, what) : launch_variant<IS_FP8, 8, 4, UE8M0, 2>(p, stream, what);
  return s.waves == 4 ? launch_variant<IS_FP8, 4, 4, UE8M0>(p, stream, what) : launch_variant<IS_FP8, 8, 4, UE8M0>(p, stream, what);
}

}  // namespace

// Waves per workgroup (the ring has four slots).  Measured (us, M = 1; 4 / 8 waves): K = 4096 -> N = 28672 INT8 27.3 / 24.8,
// K = 4096 -> N = 6144 INT8 10.7 / 10.3, K = 7168 -> N = 36864 FP8 48.9 / 48.2, K = 14336 -> N = 4096 INT8 14.5 / 15.7,
// K = 18432 -> N = 7168 FP8 27.2 / 29.8, K = 2048 -> N = 7168 FP8 7.0 / 9.2, K = 1536 -> N = 24576 FP8 11.5 / 18.1; sixteen
// waves were slower everywhere.  Eight waves up to K = 8192 (one or two turns of the ring); four for longer K and where K
// has at most 16 blocks.
WavesplitShape wavesplit_shape(int64_t K) {
  const int64_t kb = (K + KSTEP - 1) / KSTEP;
  return (kb > 16 && kb <= 64) ? WavesplitShape{8, 4} : WavesplitShape{4, 4};
}

// Two channel tiles per workgroup (32 channels, FP8): where the tokens' share of the L2 traffic outweighs the halved number of
// workgroups (the measurements stand beside the thresholds in route_constants.h).
bool wavesplit_two_tiles(bool is_fp8, int64_t M, int64_t N, int64_t K) {
  if (!is_fp8 || N % 32 != 0) return false;
  const RouteConstants& rc = route_constants();
  if ((double)(N / 32) < rc.wavesplit_two_tile_min_workgroups) return false;
  return (double)M >= rc.wavesplit_two_tile_min_tokens || (double)((K + KSTEP - 1) / KSTEP) > rc.wavesplit_two_tile_long_k_blocks;
}

bool wavesplit_supported(int64_t M, int64_t N, int64_t K) { return M >= 1 && M <= 16 && K % KSTEP == 0 && N % 16 == 0; }

int launch_fp8_wavesplit(GemmParams& p, hipStream_t stream, const char* what) { return launch_wavesplit<true>(p, stream, what); }
int launch_int8_wavesplit(GemmParams& p, hipStream_t stream, const char* what) { return launch_wavesplit<false>(p, stream, what); }
int launch_fp8_wavesplit_ue8m0(GemmParams& p, hipStream_t stream, const char* what) { return launch_wavesplit<true, true>(p, stream, what); }

}  // namespace mi355
