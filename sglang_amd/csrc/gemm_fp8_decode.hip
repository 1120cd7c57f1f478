// Decode (M <= 16) GEMMs for gfx950 - blockwise-scaled FP8 and per-token x per-channel INT8: barrier-free weight streaming.
//
// With at most 16 tokens every weight byte is used by exactly one MFMA and never again, so the kernel is bound by how
// fast the weight leaves HBM.  Measured on MI355X, a wave instruction that fetches 8 rows x 128 contiguous bytes streams
// at 6.7 TB/s, while one that fetches the MFMA operand layout directly (16 rows x 64 bytes) only reaches 5.0 TB/s.  So
// the weight is fetched in the first shape, with direct-to-LDS loads (global_load_lds_dwordx4), into a slice of LDS that
// belongs to ONE wave, and read back in operand layout by the same wave: no other wave touches the slice, so the K loop
// has no barrier.  Each wave owns 32 output channels and runs a private ring of four 4 KB stages, three K blocks always
// in flight; eight waves per CU keep ~100 KB in flight per CU.
//
// Everything else is taken out of the loop, because any ordinary load in it makes the compiler wait for ALL
// outstanding loads (the ring would collapse to depth one):
//   * a workgroup (4 waves = 128 channels = one weight scale block) works on one range of KB_PER K blocks; its tokens for
//     that range (16 x KB_PER x 128 B) are copied into LDS once, before the loop, and shared by the four waves;
//   * the token scales of the range sit in registers; the weight-block scales come by scalar loads;
//   * the workgroup then walks over several 128-channel groups with the same tokens, and the ring keeps running across
//     group boundaries, so the start-up latency is paid once per workgroup, not once per 32 KB of weight.
// The ring stages are separate __shared__ arrays and the loop is unrolled over them, so the compiler tells a load into
// one stage from reads of another and places exact vmcnt waits.  XOR swizzle and chunk mapping are those of the other
// kernels (chunks q and q + 4 per lane quarter: full-rate LDS reads).
//
// Split along K: every K range writes a partial tile to the caller's workspace and splitk_reduce_kernel adds them in a
// fixed order.  (INT8 shapes with more than one K range all take the wave-split kernel of gemm_decode_wavesplit.hip, which
// was measured faster for them at every decode size; the INT8 split variant of this kernel is therefore not built.)  INT8 uses two
// v_mfma_i32_16x16x64_i8 per K block (chunk q of both operands, then chunk q + 4) and has no scales in the loop.
// Packed UE8M0 scales on both operands (GemmParams.ue8m0): the token's exponent words of the range sit in registers, the
// weight blocks' come by scalar loads, and v_mfma_scale_f32_16x16x128_f8f6f4 applies the byte of each and accumulates in
// place, so the loop has no scale arithmetic.  The compiler sinks the last tile's MFMAs of a group into the group's guarded
// stores (only lanes of valid tokens are active there, but an MFMA reads all 64): their scale operands are therefore put
// into vector registers at the top of the group (in_vgpr).
// Requires K % 128 == 0, N % 128 == 0 and 16-byte aligned rows; other shapes take the generic kernel.
#include "gemm_common.h"

namespace mi355 {
namespace {

constexpr int KB_PER = 8;        // K blocks per workgroup range
constexpr int NT = 2;            // channel tiles of 16 per wave
constexpr int WAVE_N = 16 * NT;  // 32 channels per wave
constexpr int WAVES = 4;         // per workgroup: 128 channels
constexpr int GROUP_N = WAVES * WAVE_N;
constexpr int SLICE = WAVE_N * KSTEP;  // 4096 B per wave and ring stage
constexpr int TOK_BLOCK = 16 * KSTEP;  // 2048 B of tokens per K block

__shared__ __attribute__((aligned(1024))) uint8_t r_stage0[WAVES * SLICE];
__shared__ __attribute__((aligned(1024))) uint8_t r_stage1[WAVES * SLICE];
__shared__ __attribute__((aligned(1024))) uint8_t r_stage2[WAVES * SLICE];
__shared__ __attribute__((aligned(1024))) uint8_t r_stage3[WAVES * SLICE];
__shared__ __attribute__((aligned(1024))) uint8_t r_tok[KB_PER * TOK_BLOCK];
// The five arrays are exactly half of a CU's 160 KB, so two workgroups share a CU.  When the kernel quantizes the tokens itself,
// the token scales of the range (KB_PER x 16 floats) pass through the head of every wave's slice of stage 3, which the ring
// fills last: a wave reads its copy back before it requests its first block into that stage.

// 16 zero bytes in global memory: the source of token chunks that lie past the end of K (short last range), so that
// whatever weight block is refetched there multiplies zeros.  Not const: it must share the operands' address space.
__device__ __attribute__((aligned(16))) uint32_t r_zero16[4] = {0, 0, 0, 0};

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;
typedef const __attribute__((address_space(4))) float* cfloat_ptr;

struct Frag {
  u32x4 lo, hi;
};
__device__ __forceinline__ v8i as_v8i(const Frag& f) {
  return v8i{(int)f.lo.x, (int)f.lo.y, (int)f.lo.z, (int)f.lo.w, (int)f.hi.x, (int)f.hi.y, (int)f.hi.z, (int)f.hi.w};
}

struct DecodeState {
  const uint8_t* b_base;      // weight matrix
  uint32_t woff[WAVE_N / 8];  // byte offset of this lane's chunk in the rows of the FIRST group
  int64_t group_stride;       // bytes between consecutive 128-channel groups
  int64_t k_byte0;            // byte offset of the first K block of the range
  int wave, groups, kb_valid;
  uint32_t rd_off[NT][2];     // operand-layout read offsets inside a slice
  uint32_t tk_off[2];         // operand-layout read offsets inside a token block
};

// Direct-to-LDS loads of one K block (flattened index f = group * KB_PER + block) of this wave's 32 channels.
//
// In the K loop these loads and the waits for them are written as instructions (MANUAL = true).  The compiler's own
// bookkeeping is correct but cannot count per ring stage: it waits for every outstanding load every other step, which
// keeps the ring half empty.  The schedule is completely regular - every step issues exactly 4 loads, whether they are
// needed or not - so the wait is a constant: a stage is read when the 2 blocks issued after it (8 loads) may still be
// in flight, s_waitcnt vmcnt(8).  Anything else that counts in vmcnt between two steps (the stores of a finished
// group, the weight-scale loads of the next) only makes that wait stricter.  A stage is overwritten only after the
// MFMAs that consumed its fragments were issued, i.e. after its LDS reads returned.
template <bool MANUAL>
__device__ __forceinline__ void issue_weights(const DecodeState& s, uint8_t* stage, int f) {
  f = min(f, s.groups * KB_PER - 1);  // past the end: fetch the last block again, nobody reads it
  const int g = f / KB_PER;
  const int d = min(f - g * KB_PER, s.kb_valid - 1);  // a short last range refetches its last block (scaled by zero)
  const uint8_t* base = s.b_base + (int64_t)g * s.group_stride + s.k_byte0 + (int64_t)d * KSTEP;  // wave-uniform
  asm volatile("" : "+s"(base));  // keep it a scalar base + 32-bit lane offset
#pragma unroll
  for (int j = 0; j < WAVE_N / 8; ++j) {
    uint8_t* dst = stage + s.wave * SLICE + j * 1024;
    if constexpr (MANUAL) {
      const uint32_t lds_addr = (uint32_t)(uintptr_t)(lptr_t)dst;
      asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(s.woff[j]), "s"(base), "s"(lds_addr)
                   : "memory");  // m0 cannot be named as a clobber (the compiler reserves it and rejects the entry); no compiler-managed use of m0 lies between these statements
    } else {
      __builtin_amdgcn_global_load_lds((gptr_t)(base + s.woff[j]), (lptr_t)dst, 16, 0, 0);
    }
  }
}

// Wait until at most `younger_blocks` blocks of direct-to-LDS loads issued after the wanted one are outstanding.
template <int YOUNGER_BLOCKS>
__device__ __forceinline__ void wait_ring() {
  if constexpr (YOUNGER_BLOCKS == 2) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
  else if constexpr (YOUNGER_BLOCKS == 1) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// UE8M0 (FP8 only): `scale` and `w_scale` carry, as bits, the token's and the weight block's exponent byte of this K block in
// byte 0; the MFMA applies both and accumulates in place.
template <bool IS_FP8, bool UE8M0 = false, typename AccT>
__device__ __forceinline__ void consume(const DecodeState& s, const uint8_t* stage, int d, float scale, AccT (&acc)[NT][4],
                                        float w_scale = 0.f) {
  const uint8_t* sl = stage + s.wave * SLICE;
  Frag t;
  t.lo = *reinterpret_cast<const u32x4*>(r_tok + d * TOK_BLOCK + s.tk_off[0]);
  t.hi = *reinterpret_cast<const u32x4*>(r_tok + d * TOK_BLOCK + s.tk_off[1]);
#pragma unroll
  for (int i = 0; i < NT; ++i) {
    Frag w;
    w.lo = *reinterpret_cast<const u32x4*>(sl + s.rd_off[i][0]);
    w.hi = *reinterpret_cast<const u32x4*>(sl + s.rd_off[i][1]);
    if constexpr (UE8M0) {
      const v4f r = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(as_v8i(w), as_v8i(t), v4f{acc[i][0], acc[i][1], acc[i][2], acc[i][3]}, 0,
                                                                     0, 0, (int)__float_as_uint(w_scale), 0, (int)__float_as_uint(scale));
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][v] = r[v];
    } else if constexpr (IS_FP8) {
      const v4f part =
          __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(as_v8i(w), as_v8i(t), v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][v] = fmaf(part[v], scale, acc[i][v]);
    } else {
      v4i c = {acc[i][0], acc[i][1], acc[i][2], acc[i][3]};
      c = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{(int)w.lo.x, (int)w.lo.y, (int)w.lo.z, (int)w.lo.w},
                                                v4i{(int)t.lo.x, (int)t.lo.y, (int)t.lo.z, (int)t.lo.w}, c, 0, 0, 0);
      c = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{(int)w.hi.x, (int)w.hi.y, (int)w.hi.z, (int)w.hi.w},
                                                v4i{(int)t.hi.x, (int)t.hi.y, (int)t.hi.z, (int)t.hi.w}, c, 0, 0, 0);
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][v] = c[v];
    }
  }
}

// QUANT (FP8 only): the tokens come unquantized (p.x16, bf16 or fp16) and the workgroup quantizes the 16 x KB_PER groups of
// its K range itself, straight into the token stage, with the arithmetic of the group quantizer's reference path
// (amax floored at 1e-10, s = amax / 448, q = e4m3fn(clamp(x / s)), group_quant.hip) - so a linear layer at decode sizes
// is this kernel plus the reduce, without a quantizer launch in front.  16 lanes per group (8 elements each); codes go
// where the direct-to-LDS copy would have put them.
template <int KBP>
__device__ __forceinline__ void load_raw_tokens(const GemmParams& p, int kb_begin, u32x4 (&raw)[KBP]) {
  // (token, K block) pairs are dealt to the sixteen 16-lane rows of the workgroup, pair r + 16 j to row r: with one token
  // the eight groups are quantized by eight rows at once instead of one row doing them one after the other
  const int gl = threadIdx.x & 15, r = threadIdx.x >> 4;
#pragma unroll
  for (int j = 0; j < KBP; ++j) {
    const int pair = r + 16 * j, m = pair / KBP, d = pair % KBP;
    if (m < p.M)  // token rows past M are never stored: whatever the stage holds there will do
      raw[j] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.x16) + (int64_t)m * p.ldx +
                                               (int64_t)min(kb_begin + d, p.kb_total - 1) * KSTEP + gl * 8);
  }
}
template <int KBP>
__device__ __forceinline__ void quantize_tokens(const GemmParams& p, int kb_begin, const u32x4 (&raw)[KBP], uint8_t* tok,
                                                float* sa_lds) {
  const int gl = threadIdx.x & 15, r = threadIdx.x >> 4;
#pragma unroll
  for (int j = 0; j < KBP; ++j) {
    const int pair = r + 16 * j, m = pair / KBP, d = pair % KBP;
    if (m >= p.M) break;  // uniform over the 16-lane row, which is all the DPP reduction below involves
    float sc;
    const u32x2 codes = quantize_group_lane(raw[j], p.x_dtype, p.x_by_reciprocal != 0, sc);
    const bool valid = kb_begin + d < p.kb_total;  // blocks past the end of K: zero tokens, zero scale
    *reinterpret_cast<u32x2*>(tok + d * TOK_BLOCK + m * KSTEP + (((gl >> 1) ^ (m & 7)) << 4) + (gl & 1) * 8) =
        valid ? codes : u32x2{0u, 0u};
    if (gl < WAVES) sa_lds[gl * (SLICE / 4) + d * 16 + m] = valid ? sc : 0.f;  // one copy per wave slice (all 16 lanes hold sc)
  }
}

// SPLIT: raw partial sums to the workspace (more than one K range).
// UE8M0 (FP8 only): p.sa / p.sb point to packed exponent words (token word (m, kw) at sa[kw * sa_sk + m], channel word (n, kw)
// at sb[kw * sb_sk + n * sb_sn], byte kb & 3 of word kb >> 2 belongs to K block kb) and the MFMA applies them.
template <bool IS_FP8, bool SPLIT, bool QUANT = false, bool UE8M0 = false>
__global__ __launch_bounds__(64 * WAVES) void decode_kernel(const GemmParams p, int groups_per_wg, int wg_per_split) {
  static_assert(IS_FP8 || !QUANT, "the fused quantizer belongs to the FP8 path");
  static_assert((IS_FP8 && !QUANT) || !UE8M0, "exponent scales come with already quantized FP8 tokens");
  using AccT = typename std::conditional<IS_FP8, float, int>::type;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l16 = lane & 15, q = lane >> 4;
  const int split = blockIdx.x / wg_per_split;
  const int g_first = (blockIdx.x - split * wg_per_split) * groups_per_wg;
  const int groups_n = p.N / GROUP_N;
  const int groups = min(groups_per_wg, groups_n - g_first);
  const int kb_begin = split * KB_PER;
  const int kb_valid = min(KB_PER, p.kb_total - kb_begin);  // the last range may be short

  DecodeState s;
  s.wave = wave;
  s.groups = groups;
  s.kb_valid = kb_valid;
  s.b_base = p.b;
  s.group_stride = (int64_t)GROUP_N * p.ldb;
  s.k_byte0 = (int64_t)kb_begin * KSTEP;
  const int lrow = lane >> 3;             // row inside the 8 rows one direct-to-LDS instruction fills
  const int logical = (lane & 7) ^ lrow;  // chunk this lane fetches so that it lands swizzled by (row & 7)
#pragma unroll
  for (int j = 0; j < WAVE_N / 8; ++j) {
    const int64_t n = (int64_t)g_first * GROUP_N + wave * WAVE_N + j * 8 + lrow;  // < N: N is a multiple of 128
    s.woff[j] = (uint32_t)(n * p.ldb + logical * 16);
  }
#pragma unroll
  for (int i = 0; i < NT; ++i) {
    const int row = i * 16 + l16;
#pragma unroll
    for (int h = 0; h < 2; ++h) s.rd_off[i][h] = row * KSTEP + (((q + 4 * h) ^ (row & 7)) << 4);
  }
#pragma unroll
  for (int h = 0; h < 2; ++h) s.tk_off[h] = l16 * KSTEP + (((q + 4 * h) ^ (l16 & 7)) << 4);

  // ---- start the weight ring, then stage the tokens of this K range (all waves share them)
  u32x4 raw_tok[QUANT ? KB_PER : 1];
  if constexpr (QUANT) load_raw_tokens<KB_PER>(p, kb_begin, raw_tok);  // requested first: they are needed first
  issue_weights<false>(s, r_stage0, 0);
  issue_weights<false>(s, r_stage1, 1);
  issue_weights<false>(s, r_stage2, 2);
  if constexpr (QUANT) {
    quantize_tokens<KB_PER>(p, kb_begin, raw_tok, r_tok, reinterpret_cast<float*>(r_stage3));
  } else {
#pragma unroll
    for (int e = 0; e < 2 * KB_PER / WAVES; ++e) {  // 16 instructions of 8 rows x 128 B, 4 per wave
      const int inst = wave * (2 * KB_PER / WAVES) + e;
      const int d = inst >> 1, half = inst & 1;
      const int m = min(half * 8 + lrow, p.M - 1);           // rows past M repeat the last token, never stored
      const uint8_t* src = p.a + (int64_t)m * p.lda + (int64_t)(kb_begin + d) * KSTEP + logical * 16;
      if (kb_begin + d >= p.kb_total) src = reinterpret_cast<const uint8_t*>(r_zero16);  // blocks past K: zeros
      __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(r_tok + d * TOK_BLOCK + half * 1024), 16, 0, 0);
    }
  }
  // FP8: token scales of the range (blocks past the end of K multiply zero tokens; their scale is set to zero too)
  float sa_r[KB_PER];
  if constexpr (QUANT) {
    __syncthreads();  // codes and scales of the range are in LDS
#pragma unroll
    for (int d = 0; d < KB_PER; ++d) sa_r[d] = reinterpret_cast<const float*>(r_stage3 + wave * SLICE)[d * 16 + l16];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // read back before this wave's first request into stage 3
  } else if constexpr (IS_FP8) {
    const float* sa_row = p.sa + (int64_t)min(l16, p.M - 1) * p.sa_sm;
#pragma unroll
    for (int d = 0; d < KB_PER; ++d) {
      const int kbc = min(kb_begin + d, p.kb_total - 1);
      if constexpr (UE8M0) {  // the block's byte of the token's word, in byte 0 (blocks past K multiply zero tokens)
        sa_r[d] = __uint_as_float(__float_as_uint(sa_row[(int64_t)(kbc >> 2) * p.sa_sk]) >> ((kbc & 3) * 8));
      } else {
        const float v = sa_row[(int64_t)kbc * p.sa_sk];
        sa_r[d] = d < kb_valid ? v : 0.f;
      }
    }
  } else {
#pragma unroll
    for (int d = 0; d < KB_PER; ++d) sa_r[d] = 0.f;
  }
  if constexpr (!QUANT) __syncthreads();  // the only barrier: tokens are in LDS

  const bool vec_ok = ((p.ldo & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
  // FP8 weight-block scales: one per K block and 128-channel group; fetched one group ahead so that using them never
  // has to wait for loads younger than the ring's
  float sb_cur[KB_PER], sb_nxt[KB_PER];
  auto load_sb = [&](int g, float (&dst)[KB_PER]) {
    if constexpr (UE8M0) {
      // one word row per weight ROW (constant over the 128-channel group): the group's first row; scalar loads
      const cfloat_ptr sb_row = (cfloat_ptr)(p.sb + (int64_t)(g_first + min(g, groups - 1)) * GROUP_N * p.sb_sn);
#pragma unroll
      for (int d = 0; d < KB_PER; ++d) {
        const int kbc = kb_begin + min(d, kb_valid - 1);
        dst[d] = __uint_as_float(__float_as_uint(sb_row[(int64_t)(kbc >> 2) * p.sb_sk]) >> ((kbc & 3) * 8));
      }
    } else if constexpr (IS_FP8) {
      // uniform addresses through a constant-address-space pointer: scalar loads, which do not count in vmcnt, so the
      // copy of these values at the end of a group never waits for the weight ring
      const cfloat_ptr sb_row =
          (cfloat_ptr)(p.sb + (int64_t)(g_first + min(g, groups - 1)) * p.sb_sn + (int64_t)kb_begin * p.sb_sk);
#pragma unroll
      for (int d = 0; d < KB_PER; ++d) dst[d] = sb_row[(int64_t)min(d, kb_valid - 1) * p.sb_sk];
    } else {
#pragma unroll
      for (int d = 0; d < KB_PER; ++d) dst[d] = 0.f;
    }
  };
  load_sb(0, sb_cur);
  for (int g = 0; g < groups; ++g) {
    const int nb = g_first + g;  // 128 channels = one weight scale block
    load_sb(g + 1, sb_nxt);
    float sc[KB_PER], wsc[KB_PER];  // fp32 scales: sc = token scale x block scale; UE8M0: the two exponent bytes apart
#pragma unroll
    for (int d = 0; d < KB_PER; ++d) {
      sc[d] = UE8M0 ? sa_r[d] : sa_r[d] * sb_cur[d];
      // UE8M0: in a vector register before the group's guarded stores (the last MFMAs may be sunk into them)
      wsc[d] = UE8M0 ? __uint_as_float((uint32_t)in_vgpr((int)__float_as_uint(sb_cur[d]))) : 0.f;
    }
#pragma unroll
    for (int d = 0; d < KB_PER; ++d) sb_cur[d] = sb_nxt[d];
    AccT acc[NT][4];
#pragma unroll
    for (int i = 0; i < NT; ++i)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][v] = 0;

    const int f0 = g * KB_PER;
#pragma unroll
    for (int d = 0; d < KB_PER; d += 4) {
      // each step: request the block three ahead into the stage consumed in the previous step, wait for the block
      // that is due (the two requested after it may still be in flight), multiply it
      issue_weights<true>(s, r_stage3, f0 + d + 3);
      wait_ring<2>();
      consume<IS_FP8, UE8M0>(s, r_stage0, d + 0, sc[d + 0], acc, wsc[d + 0]);
      __builtin_amdgcn_sched_barrier(0);
      issue_weights<true>(s, r_stage0, f0 + d + 4);
      wait_ring<2>();
      consume<IS_FP8, UE8M0>(s, r_stage1, d + 1, sc[d + 1], acc, wsc[d + 1]);
      __builtin_amdgcn_sched_barrier(0);
      issue_weights<true>(s, r_stage1, f0 + d + 5);
      wait_ring<2>();
      consume<IS_FP8, UE8M0>(s, r_stage2, d + 2, sc[d + 2], acc, wsc[d + 2]);
      __builtin_amdgcn_sched_barrier(0);
      issue_weights<true>(s, r_stage2, f0 + d + 6);
      wait_ring<2>();
      consume<IS_FP8, UE8M0>(s, r_stage3, d + 3, sc[d + 3], acc, wsc[d + 3]);
      __builtin_amdgcn_sched_barrier(0);
    }

    if (g == groups - 1) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no ring refetch may outlive the workgroup's LDS
    // ---- lane holds channels 16 i + 4q .. +3 of this wave's 32, for token l16
    if (l16 < p.M) {
#pragma unroll
      for (int i = 0; i < NT; ++i) {
        const int n = nb * GROUP_N + wave * WAVE_N + i * 16 + 4 * q;
        if constexpr (SPLIT) {
          AccT* wsp = reinterpret_cast<AccT*>(p.ws) + ((int64_t)split * p.M + l16) * p.N + n;
#pragma unroll
          for (int v = 0; v < 4; ++v) wsp[v] = acc[i][v];
        } else if constexpr (IS_FP8) {
          fp8_channel_epilogue(p, n, acc[i]);
          store_out4(p.out, p.out_dtype, (int64_t)l16 * p.ldo + n, acc[i], 4, vec_ok);
        } else if (p.out_dtype == MI355_I32) {
          int* o = reinterpret_cast<int*>(p.out) + (int64_t)l16 * p.ldo + n;
#pragma unroll
          for (int v = 0; v < 4; ++v) o[v] = acc[i][v];
        } else {
          const float sa_m = p.sa[l16];
          float r[4];
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            float t = mul_rn((float)acc[i][v], mul_rn(p.sb[n + v], sa_m));
            if (p.bias) {
              const uint32_t hb = reinterpret_cast<const uint16_t*>(p.bias)[n + v];
              t = add_rn(t, (p.out_dtype == MI355_BF16) ? bf16_bits_to_f32(hb) : f16_bits_to_f32(hb));
            }
            r[v] = t;
          }
          store_out4(p.out, p.out_dtype, (int64_t)l16 * p.ldo + n, r, 4, vec_ok);
        }
      }
    }
  }
}

}  // namespace

// The decode kernel splits K into ranges of KB_PER blocks.
int decode_splits(int64_t M, int64_t N, int64_t K) {
  const int64_t kb_total = (K + KSTEP - 1) / KSTEP;
  return (int)((kb_total + KB_PER - 1) / KB_PER);
}

int decode_kb_per_range() { return KB_PER; }

// Shapes the decode kernel takes: one token tile, whole K blocks, channels in whole groups of 128.
bool decode_supported(int64_t M, int64_t N, int64_t K) { return M >= 1 && M <= 16 && K % KSTEP == 0 && N % GROUP_N == 0; }

// Also needs 16-byte aligned rows and row offsets below 4 GiB.  The caller sets p.splits (= decode_splits) and p.ws.
// About two workgroups per CU; each walks this many consecutive channel groups with the same tokens.
int decode_groups_per_wg(int64_t N, int splits) {
  const int gpw = (int)(((N / GROUP_N) * splits + 511) / 512);
  return gpw < 1 ? 1 : gpw;
}

template <bool IS_FP8>
static int launch_decode(GemmParams& p, int gpw, hipStream_t stream, const char* what) {
  const int groups_n = p.N / GROUP_N;
  const int wg_per_split = (groups_n + gpw - 1) / gpw;
  p.tiles_m = 1;
  p.tiles_n = groups_n;
  const dim3 grid((unsigned)(wg_per_split * p.splits));
  if constexpr (IS_FP8) {
    if (p.x16 != nullptr) {  // tokens arrive unquantized
      if (p.splits > 1)
        hipLaunchKernelGGL((decode_kernel<true, true, true>), grid, dim3(64 * WAVES), 0, stream, p, gpw, wg_per_split);
      else
        hipLaunchKernelGGL((decode_kernel<true, false, true>), grid, dim3(64 * WAVES), 0, stream, p, gpw, wg_per_split);
      return check_launch(what);
    }
  }
  if (p.splits > 1) {
    if constexpr (IS_FP8) {
      hipLaunchKernelGGL((decode_kernel<true, true>), grid, dim3(64 * WAVES), 0, stream, p, gpw, wg_per_split);
    } else {
      // INT8 shapes with more than one K range (8 blocks) all go to the wave-split kernel: this variant is not built
      set_error("%s: the INT8 streaming decode kernel has no K split", what);
      return MI355_ERR_UNSUPPORTED;
    }
  } else {
    hipLaunchKernelGGL((decode_kernel<IS_FP8, false>), grid, dim3(64 * WAVES), 0, stream, p, gpw, wg_per_split);
  }
  return check_launch(what);
}

int launch_fp8_decode(GemmParams& p, int gpw, hipStream_t stream, const char* what) {
  if (p.ue8m0) {  // packed exponent words on both operands, applied by the MFMA
    const int groups_n = p.N / GROUP_N;
    const int wg_per_split = (groups_n + gpw - 1) / gpw;
    p.tiles_m = 1;
    p.tiles_n = groups_n;
    const dim3 grid((unsigned)(wg_per_split * p.splits));
    if (p.splits > 1)
      hipLaunchKernelGGL((decode_kernel<true, true, false, true>), grid, dim3(64 * WAVES), 0, stream, p, gpw, wg_per_split);
    else
      hipLaunchKernelGGL((decode_kernel<true, false, false, true>), grid, dim3(64 * WAVES), 0, stream, p, gpw, wg_per_split);
    return check_launch(what);
  }
  return launch_decode<true>(p, gpw, stream, what);
}
int launch_int8_decode(GemmParams& p, int gpw, hipStream_t stream, const char* what) { return launch_decode<false>(p, gpw, stream, what); }

}  // namespace mi355
