// Small-M (decode) blockwise-scaled FP8 GEMM for gfx950: barrier-free weight streaming.
//
// With at most 64 tokens every weight byte is used once per token tile and never again, so the kernel is bound by how
// fast the weight leaves HBM.  Measured on MI355X, a wave instruction that fetches 8 rows x 128 contiguous bytes streams
// at 6.7 TB/s, while one that fetches the MFMA operand layout directly (16 rows x 64 bytes) only reaches 5.0 TB/s.  So
// the weight is fetched in the first shape, with direct-to-LDS loads (global_load_lds_dwordx4), into a slice of LDS that
// belongs to ONE wave, and read back in operand layout by the same wave.  No other wave touches the slice, so there is
// no barrier anywhere: each wave owns 32 output channels and a range of K blocks and runs a private ring of RING
// stages, always RING - 1 K blocks (RING - 1 x 4 KB) in flight.  With 8 waves per CU that is ~100 KB in flight per CU,
// enough to cover HBM latency at full bandwidth.
//
// The ring stages are separate __shared__ arrays and the loop is unrolled over them, so the compiler can tell a load
// into one stage from reads of another and places precise vmcnt waits.  Tokens (a few KB per K block, shared by every
// wave) and scales come through the caches with ordinary loads, one K block ahead.  XOR swizzle and chunk mapping are
// the ones of the other kernels (chunks q and q + 4 per lane quarter: full-rate LDS reads).
//
// Split along K: partial tiles go to the caller's workspace and splitk_reduce_kernel adds them in a fixed order.
#include "gemm_common.h"

namespace mi355 {
namespace {

constexpr int RING = 4;          // LDS stages per wave
constexpr int NT = 2;            // channel tiles of 16 per wave
constexpr int WAVE_N = 16 * NT;  // 32 channels per wave
constexpr int WAVES = 4;         // per workgroup
constexpr int SLICE = WAVE_N * KSTEP;  // 4096 B per wave and stage

__shared__ __attribute__((aligned(1024))) uint8_t r_stage0[WAVES * SLICE];
__shared__ __attribute__((aligned(1024))) uint8_t r_stage1[WAVES * SLICE];
__shared__ __attribute__((aligned(1024))) uint8_t r_stage2[WAVES * SLICE];
__shared__ __attribute__((aligned(1024))) uint8_t r_stage3[WAVES * SLICE];

// source of 16-byte chunks past the end of K (K % 128 != 0); deliberately not const: it must live in the same (global)
// address space as the operands, or selecting between the two addresses would turn the loads into FLAT loads
__device__ __attribute__((aligned(16))) uint32_t r_zero16[4] = {0, 0, 0, 0};

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

struct Frag {
  u32x4 lo, hi;
};
__device__ __forceinline__ v8i as_v8i(const Frag& f) {
  return v8i{(int)f.lo.x, (int)f.lo.y, (int)f.lo.z, (int)f.lo.w, (int)f.hi.x, (int)f.hi.y, (int)f.hi.z, (int)f.hi.w};
}

template <int MT>
struct DecodeState {
  const uint8_t* wsrc[WAVE_N / 8];  // per direct-to-LDS instruction: this lane's row start + 16 * its logical chunk
  int chunk_byte;                   // 16 * that logical chunk (for the K tail)
  const uint8_t* trow[MT];          // token rows (+ 16 q)
  const float* sa_row[MT];
  const float* sb_row;
  int64_t sa_sk, sb_sk;
  int K, kb_total, kb_end;
  bool lo_ok_last, hi_ok_last;
  uint32_t rd_off[NT][2];  // operand-layout read offsets inside a slice
  int wave;
};

// KFULL: K is a multiple of 128, every chunk of every block lies inside its row.
template <int MT, bool KFULL>
__device__ __forceinline__ void issue_weights(const DecodeState<MT>& s, uint8_t* stage, int kb) {
  kb = min(kb, s.kb_end - 1);  // past the range: fetch the last block again, nobody reads it
#pragma unroll
  for (int j = 0; j < WAVE_N / 8; ++j) {
    const uint8_t* src = s.wsrc[j] + (int64_t)kb * KSTEP;
    if constexpr (!KFULL) {
      if (kb * KSTEP + s.chunk_byte >= s.K) src = reinterpret_cast<const uint8_t*>(r_zero16);
    }
    __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(stage + s.wave * SLICE + j * 1024), 16, 0, 0);
  }
}

// Branch-free on purpose: a conditional load would put control flow into the K loop and make the compiler fall back to
// waiting for every outstanding load.  Past the end of K the ADDRESS is redirected to a block of zeros; a block past
// this wave's range is refetched and weighted with zero.
template <int MT, bool KFULL>
__device__ __forceinline__ void load_tokens(const DecodeState<MT>& s, int kb, Frag (&t)[MT], float (&sc)[MT + 1]) {
  kb = min(kb, s.kb_end - 1);
  const int64_t off = (int64_t)kb * KSTEP;
  // raw values only: multiplying here would make the wave wait for these loads in the step that issues them
  sc[MT] = s.sb_row[(int64_t)kb * s.sb_sk];
  bool lo_ok = true, hi_ok = true;
  if constexpr (!KFULL) {
    const bool last = kb == s.kb_total - 1;
    lo_ok = !last || s.lo_ok_last, hi_ok = !last || s.hi_ok_last;
  }
  const uint8_t* zero = reinterpret_cast<const uint8_t*>(r_zero16);
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    t[j].lo = *reinterpret_cast<const u32x4*>(lo_ok ? s.trow[j] + off : zero);
    t[j].hi = *reinterpret_cast<const u32x4*>(hi_ok ? s.trow[j] + off + 64 : zero);
    sc[j] = s.sa_row[j][(int64_t)kb * s.sa_sk];
  }
}

template <int MT>
__device__ __forceinline__ void consume(const DecodeState<MT>& s, const uint8_t* stage, bool valid, const Frag (&t)[MT],
                                        const float (&sc)[MT + 1], float (&acc)[NT][MT][4]) {
  const uint8_t* sl = stage + s.wave * SLICE;
  float scale[MT];
#pragma unroll
  for (int j = 0; j < MT; ++j) scale[j] = valid ? sc[j] * sc[MT] : 0.f;  // sa[m, kb] * sb[nb, kb]; nothing past the range
#pragma unroll
  for (int i = 0; i < NT; ++i) {
    Frag w;
    w.lo = *reinterpret_cast<const u32x4*>(sl + s.rd_off[i][0]);
    w.hi = *reinterpret_cast<const u32x4*>(sl + s.rd_off[i][1]);
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      const v4f part = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(as_v8i(w), as_v8i(t[j]), v4f{0.f, 0.f, 0.f, 0.f},
                                                                       0, 0, 0, 0, 0, 0);
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = fmaf(part[v], scale[j], acc[i][j][v]);
    }
  }
}

// MT: token tiles of 16 (M <= 16 * MT).  SPLIT: raw partial sums to the workspace.
template <int MT, bool SPLIT, bool KFULL>
__global__ __launch_bounds__(64 * WAVES) void fp8_decode_kernel(const GemmParams p) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: keeps the K bookkeeping on the scalar unit
  const int l16 = lane & 15, q = lane >> 4;
  const int tiles_n = p.tiles_n;  // ceil(N / 32)
  const int wid = blockIdx.x * WAVES + wave;
  if (wid >= tiles_n * p.splits) return;  // whole waves only: there is no barrier in this kernel
  const int split = wid / tiles_n;
  const int n0 = (wid - split * tiles_n) * WAVE_N;
  const int kb_begin = split * p.kb_per_split;

  DecodeState<MT> s;
  s.wave = wave;
  s.K = p.K;
  s.kb_total = p.kb_total;
  s.kb_end = min(p.kb_total, kb_begin + p.kb_per_split);
  {
    const int lrow = lane >> 3;               // row inside the 8 rows one instruction fills
    const int logical = (lane & 7) ^ lrow;    // chunk this lane fetches so that it lands swizzled by (row & 7)
    s.chunk_byte = logical * 16;
#pragma unroll
    for (int j = 0; j < WAVE_N / 8; ++j)
      s.wsrc[j] = p.b + (int64_t)min(n0 + j * 8 + lrow, p.N - 1) * p.ldb + s.chunk_byte;
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      const int row = i * 16 + l16;
#pragma unroll
      for (int h = 0; h < 2; ++h) s.rd_off[i][h] = row * KSTEP + (((q + 4 * h) ^ (row & 7)) << 4);
    }
  }
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    const int m = min(j * 16 + l16, p.M - 1);
    s.trow[j] = p.a + (int64_t)m * p.lda + q * 16;
    s.sa_row[j] = p.sa + (int64_t)m * p.sa_sm;
  }
  // 32 channels starting at a multiple of 32 lie inside one 128-wide scale block
  s.sb_row = p.sb + (int64_t)(min(n0, p.N - 1) / 128) * p.sb_sn;
  s.sa_sk = p.sa_sk;
  s.sb_sk = p.sb_sk;
  s.lo_ok_last = (p.kb_total - 1) * KSTEP + q * 16 < p.K;
  s.hi_ok_last = (p.kb_total - 1) * KSTEP + q * 16 + 64 < p.K;

  float acc[NT][MT][4];
#pragma unroll
  for (int i = 0; i < NT; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.f;

  // ---- fill the ring, fetch the first token fragments
  issue_weights<MT, KFULL>(s, r_stage0, kb_begin + 0);
  issue_weights<MT, KFULL>(s, r_stage1, kb_begin + 1);
  issue_weights<MT, KFULL>(s, r_stage2, kb_begin + 2);
  Frag ta[MT], tb[MT];
  float sca[MT + 1], scb[MT + 1];  // token scales of the block, then the weight-block scale
  load_tokens<MT, KFULL>(s, kb_begin, ta, sca);

  // ---- RING blocks per trip; blocks past kb_end are computed on refetched data and weighted with zero
  for (int kb = kb_begin; kb < s.kb_end; kb += RING) {
    issue_weights<MT, KFULL>(s, r_stage3, kb + 3);
    load_tokens<MT, KFULL>(s, kb + 1, tb, scb);
    consume<MT>(s, r_stage0, true, ta, sca, acc);
    __builtin_amdgcn_sched_barrier(0);
    issue_weights<MT, KFULL>(s, r_stage0, kb + 4);
    load_tokens<MT, KFULL>(s, kb + 2, ta, sca);
    consume<MT>(s, r_stage1, kb + 1 < s.kb_end, tb, scb, acc);
    __builtin_amdgcn_sched_barrier(0);
    issue_weights<MT, KFULL>(s, r_stage1, kb + 5);
    load_tokens<MT, KFULL>(s, kb + 3, tb, scb);
    consume<MT>(s, r_stage2, kb + 2 < s.kb_end, ta, sca, acc);
    __builtin_amdgcn_sched_barrier(0);
    issue_weights<MT, KFULL>(s, r_stage2, kb + 6);
    load_tokens<MT, KFULL>(s, kb + 4, ta, sca);
    consume<MT>(s, r_stage3, kb + 3 < s.kb_end, tb, scb, acc);
    __builtin_amdgcn_sched_barrier(0);
  }

  // ---- lane holds channels n0 + 16 i + 4q .. +3 of token 16 j + l16
  const bool vec_ok = ((p.ldo & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
#pragma unroll
  for (int i = 0; i < NT; ++i) {
    const int n = n0 + i * 16 + 4 * q;
    if (n >= p.N) continue;
    const int nvalid = min(4, p.N - n);
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      const int m = j * 16 + l16;
      if (m >= p.M) continue;
      if constexpr (SPLIT) {
        float* wsp = reinterpret_cast<float*>(p.ws) + ((int64_t)split * p.M + m) * p.N + n;
#pragma unroll
        for (int v = 0; v < 4; ++v)
          if (v < nvalid) wsp[v] = acc[i][j][v];
      } else {
        store_out4(p.out, p.out_dtype, (int64_t)m * p.ldo + n, acc[i][j], nvalid, vec_ok);
      }
    }
  }
}

template <int MT>
void launch_mt(const GemmParams& p, hipStream_t stream) {
  const unsigned waves = (unsigned)(p.tiles_n * p.splits);
  const dim3 grid((waves + WAVES - 1) / WAVES);
  const bool kfull = p.K % KSTEP == 0;
  if (p.splits > 1) {
    if (kfull) hipLaunchKernelGGL((fp8_decode_kernel<MT, true, true>), grid, dim3(64 * WAVES), 0, stream, p);
    else hipLaunchKernelGGL((fp8_decode_kernel<MT, true, false>), grid, dim3(64 * WAVES), 0, stream, p);
  } else {
    if (kfull) hipLaunchKernelGGL((fp8_decode_kernel<MT, false, true>), grid, dim3(64 * WAVES), 0, stream, p);
    else hipLaunchKernelGGL((fp8_decode_kernel<MT, false, false>), grid, dim3(64 * WAVES), 0, stream, p);
  }
}

}  // namespace

// Split count for the decode kernel: about 16 waves per CU, and at least two ring trips of K blocks per wave.
int decode_splits(int64_t M, int64_t N, int64_t K) {
  const int64_t kb_total = (K + KSTEP - 1) / KSTEP;
  const int64_t tiles_n = (N + WAVE_N - 1) / WAVE_N;
  if (N % 4 != 0) return 1;  // the reduce kernel works on aligned quads of one row
  int64_t want = (4096 + tiles_n - 1) / tiles_n;
  const int64_t max_by_k = kb_total / (2 * RING) > 0 ? kb_total / (2 * RING) : 1;
  if (want > max_by_k) want = max_by_k;
  if (want > 64) want = 64;
  if (want < 1) want = 1;
  const int64_t per = (kb_total + want - 1) / want;
  return (int)((kb_total + per - 1) / per);
}

// M <= 64 supported (the dispatcher uses it up to 16), 16-byte aligned rows, K % 16 == 0.  p.splits / p.kb_per_split / p.ws are set by the caller.
int launch_fp8_decode(GemmParams& p, hipStream_t stream, const char* what) {
  p.tiles_m = 1;
  p.tiles_n = (p.N + WAVE_N - 1) / WAVE_N;
  if (p.M <= 16) launch_mt<1>(p, stream);
  else if (p.M <= 32) launch_mt<2>(p, stream);
  else launch_mt<4>(p, stream);
  return check_launch(what);
}

}  // namespace mi355
