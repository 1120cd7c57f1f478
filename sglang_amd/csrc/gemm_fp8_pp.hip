// Large-M blockwise-scaled FP8 GEMM for gfx950: 256 x 256 macro tile, 8 waves, two-phase ("ping-pong") schedule.
//
// What the counters of a kernel that interleaves everything say: with the MFMAs, the promotion FMAs, the LDS operand
// reads and the direct-to-LDS loads of the next K block mixed into one instruction stream per wave, the matrix pipe is
// busy 53 % of the time.  Taking the loads out (nothing else changed) brings it to 94 %; making them hit in L2 or never
// waiting for them changes little.  A wave issues in order, so whenever one of its vector-memory instructions has to wait
// for a slot in the address path the MFMAs behind it wait too, and with two such waves per SIMD both are often stuck.
//
// So the two waves of a SIMD take turns.  Waves 0..3 (token rows 0..127 of the tile) and waves 4..7 (rows 128..255) sit
// one per SIMD each; while one group runs a COMPUTE phase - sixteen MFMAs with their promotion FMAs, operands already in
// registers, nothing else - the other runs a MEMORY phase: LDS operand reads for its next compute phase, the direct-to-LDS
// loads of the next K block, scale fetches.  A workgroup barrier ends every phase; group 1 starts one phase late, so the
// groups alternate and the matrix pipe of every SIMD always has exactly one wave feeding it.
//
// One K block (128 bytes of K) per wave = 32 MFMAs (v_mfma_f32_16x16x128_f8f6f4) = two compute phases of four token tiles
// x four channel tiles, each preceded by a memory phase that copies its operands from LDS into registers:
//   M0(k): weight fragments + token tiles 0..3 of block k -> registers        C0(k): 16 MFMAs / 64 FMAs
//   M1(k): token tiles 4..7 -> registers                                       C1(k): 16 MFMAs / 64 FMAs
// Because operands leave LDS a phase before they are used, a 64-row band of a stage is free again long before the block
// is finished, and its successor (block k + 2, same stage) can be requested early.  Measured on this part: LDS reads a
// wave issues behind its own direct-to-LDS loads return ~65 cycles later per load in front of them, so inside a memory
// phase the LDS reads go first and the loads last.  Every wave fetches one 8-row slice of every band:
//   set A(b) = token scales, the four channel bands, token rows 0..63 and 128..191 of block b: requested in M1(b - 2),
//              when both groups have copied those rows of block b - 2 out (M0 phases); needed from M0(b) of group 0 on;
//   set B(b) = token rows 64..127 and 192..255: requested in M0(b - 1), after the M1 phases that read them; needed
//              from M1(b) of group 0 on.
// Loads complete in order, so "set X has landed" is a constant count: at the end of every memory phase exactly nine
// younger loads may still be in flight (s_waitcnt vmcnt(9)), and each set has four phases - a whole K block - to land.
// Token scales: measured, ONE 4-byte-per-lane load per wave and K block (direct-to-LDS or to a register, whatever its
// address or position in the stream) makes this kernel 1.5x slower, while 16-byte-per-lane loads stream freely.  So the
// scales must be M-major (256 consecutive floats per tile and K block, the layout fp8_blockwise_scaled_mm prescribes),
// and each wave fetches 32 of them with the first eight lanes of a 16-byte direct-to-LDS load; the dispatcher re-lays
// other layouts out into the workspace first.  They use four small LDS stages so that they can travel with set A.
// Loads, waits and barriers are written as instructions (the compiler would wait for all loads at every barrier).
// Arithmetic, operand roles, LDS layout and swizzle are those of gemm_w8a8.hip.
#include "gemm_common.h"

namespace mi355 {
namespace {

constexpr int SM_BLOCK_F32 = 0, SM_UE8M0 = 1, SM_EPILOGUE = 2;
constexpr int G_THREADS = 512;
constexpr int G_BM = 256, G_BN = 256, G_WM = 128, G_WN = 64;
constexpr int G_MT = G_WM / 16, G_NT = G_WN / 16;  // 8 token tiles x 4 channel tiles per wave
constexpr int G_HT = G_MT / 2;                     // token tiles per compute phase
constexpr int G_ROWS = G_BM + G_BN;
constexpr int G_LOADS = G_ROWS / 64;               // 8 direct-to-LDS tile loads per wave and K block
constexpr int G_STAGE = G_ROWS * KSTEP;

// the two stages are one array: after the K loop it holds the output tile on its way to memory
__shared__ __attribute__((aligned(1024))) uint8_t g_stages[2 * G_STAGE];
#define g_stage0 (g_stages)
#define g_stage1 (g_stages + G_STAGE)
static_assert(2 * G_STAGE >= OUT_TILE_BYTES, "the output tile is staged in the two input stages");
// token scales: four stages (block b in stage b % 4) of 256 floats
__shared__ __attribute__((aligned(256))) float g_scale[4 * G_BM];

__device__ __attribute__((aligned(16))) uint32_t g_zero16[4] = {0, 0, 0, 0};  // source of chunks past the end of K

typedef __attribute__((address_space(3))) void* lptr_t;
typedef const __attribute__((address_space(4))) float* cfloat_ptr;
typedef const __attribute__((address_space(3))) uint8_t* lds_cptr;

__device__ __forceinline__ u32x4 lds16(lds_cptr p, int imm) {
  return *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(p + imm);
}

struct Frag {
  u32x4 lo, hi;
};
__device__ __forceinline__ v8i as_v8i(const Frag& f) {
  return v8i{(int)f.lo.x, (int)f.lo.y, (int)f.lo.z, (int)f.lo.w, (int)f.hi.x, (int)f.hi.y, (int)f.hi.z, (int)f.hi.w};
}

struct PpState {
  const uint8_t* a_base;
  const uint8_t* b_base;
  uint32_t goff[G_LOADS];  // lane's byte offset from the matrix base (rows clamped); loads 0..3 token rows, 4..7 channel rows
  int chunk_byte;          // 16 * logical chunk this lane fetches
  const float* sa_base;    // token scales, M-major: element (m, kb) at sa_base[kb * sa_sk + m]
  uint32_t sa_off;         // byte offset of the four scales this lane fetches (lanes 0..7), clamped to the last valid quad
  cfloat_ptr sb_ptr;       // &sb[nb, 0] of this wave's 128-channel block
  int64_t sa_sk, sb_sk;
  int K, wave, kb_last;
  uint32_t tok_off[2], ch_off[2], sc_off;
};

// Direct-to-LDS load number i (< 8) of K block kb (clamped to the last block): tile rows i * 64 + 8 * wave .. + 7 into
// `stage`.  Written as instructions so that the compiler does not count them.  They write m0 (it cannot be named as a
// clobber: reserved register); no compiler-managed use of m0 lies between these statements.
template <bool KFULL>
__device__ __forceinline__ void issue_one(const PpState& s, int i, uint8_t* stage, int kb) {
  kb = min(kb, s.kb_last);
  const uint8_t* base = (i < G_LOADS / 2 ? s.a_base : s.b_base) + (uint64_t)kb * KSTEP;  // wave-uniform
  const uint32_t lds_addr = (uint32_t)(uintptr_t)(lptr_t)(stage + (i * 64 + s.wave * 8) * KSTEP);
  if constexpr (KFULL) {
    asm volatile("" : "+s"(base));
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(s.goff[i]), "s"(base), "s"(lds_addr) : "memory");
  } else {
    // K ends inside the last block: chunks past the end come from a block of zeros (per-lane 64-bit addresses)
    const uint8_t* src = base + s.goff[i];
    if (kb * KSTEP + s.chunk_byte >= s.K) src = reinterpret_cast<const uint8_t*>(g_zero16);
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds_addr) : "memory");
  }
}

// The wave's 32 token scales of block b (tokens 32 * wave .. + 31 of the tile) into scale stage b % 4: lanes 0..7 fetch
// 16 bytes each.  exec is narrowed and restored inside the statement.
template <bool UE8M0>
__device__ __forceinline__ void issue_scales(const PpState& s, int b) {
  // fp32 scales: one row of floats per K block; packed exponents: one row of 32-bit words per four K blocks (fetched
  // again for each of the four, which keeps the load count per K block constant)
  const int srow = UE8M0 ? (min(b, s.kb_last) >> 2) : min(b, s.kb_last);
  const float* base = s.sa_base + (int64_t)srow * s.sa_sk;  // wave-uniform
  asm volatile("" : "+s"(base));
  const uint32_t lds_addr = (uint32_t)(uintptr_t)(lptr_t)(g_scale + (b & 3) * G_BM + s.wave * 32);
  uint64_t saved;
  asm volatile(
      "s_mov_b64 %0, exec\n\ts_mov_b64 exec, 0xff\n\ts_mov_b32 m0, %3\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b64 exec, %0"
      : "=&s"(saved)
      : "v"(s.sa_off), "s"(base), "s"(lds_addr)
      : "memory");
}

// Set A of block b: scales, channel bands, token rows 0..63 and 128..191 (7 loads).  Set B: token rows 64..127, 192..255.
constexpr int SET_A = 7, SET_B = 2;
template <bool KFULL, bool UE8M0>
__device__ __forceinline__ void issue_set_a(const PpState& s, uint8_t* stage, int b) {
  issue_scales<UE8M0>(s, b);
#pragma unroll
  for (int i = 4; i < 8; ++i) issue_one<KFULL>(s, i, stage, b);
  issue_one<KFULL>(s, 0, stage, b);
  issue_one<KFULL>(s, 2, stage, b);
}
template <bool KFULL>
__device__ __forceinline__ void issue_set_b(const PpState& s, uint8_t* stage, int b) {
  issue_one<KFULL>(s, 1, stage, b);
  issue_one<KFULL>(s, 3, stage, b);
}

// End of a compute phase.
__device__ __forceinline__ void compute_end() {
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_setprio(2);  // the memory phase that follows runs above the other group's MFMA stream (measured: ~1 %)
  asm volatile("s_barrier" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

// End of a memory phase: its LDS reads have returned (the compute phase that follows must not start with a wait) and
// all but the nine youngest of this wave's loads have landed.
__device__ __forceinline__ void memory_end() {
  static_assert(SET_A + SET_B == 9, "the wait is written for nine loads per K block");
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_waitcnt vmcnt(9) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  __builtin_amdgcn_s_setprio(0);
  __builtin_amdgcn_sched_barrier(0);
}

// Memory phase, operand part: token tiles 4 * HALF .. + 3 of `cur` (and, for HALF == 0, the four weight fragments)
// into registers; their scales times the weight-block scale.
// SM_UE8M0: scb[jj] carries (as bits) the token's packed exponent word shifted so that the byte of this K block is byte 0;
// SM_EPILOGUE: the exponent byte of 1.0.
template <int HALF, int SM>
__device__ __forceinline__ void read_operands(const PpState& s, const uint8_t* cur, const float* sc_cur, float sbv, int kb,
                                              Frag (&w)[G_NT], Frag (&tok)[G_HT], float (&scb)[G_HT]) {
  const lds_cptr ch0 = (lds_cptr)cur + s.ch_off[0], ch1 = (lds_cptr)cur + s.ch_off[1];
  const lds_cptr tk0 = (lds_cptr)cur + s.tok_off[0], tk1 = (lds_cptr)cur + s.tok_off[1];
  const float* scp = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(sc_cur) + s.sc_off);
  if constexpr (HALF == 0) {
#pragma unroll
    for (int i = 0; i < G_NT; ++i) {
      w[i].lo = lds16(ch0, i * 2048);
      w[i].hi = lds16(ch1, i * 2048);
    }
  }
#pragma unroll
  for (int jj = 0; jj < G_HT; ++jj) {
    tok[jj].lo = lds16(tk0, (HALF * G_HT + jj) * 2048);
    tok[jj].hi = lds16(tk1, (HALF * G_HT + jj) * 2048);
  }
#pragma unroll
  for (int jj = 0; jj < G_HT; ++jj) {
    if constexpr (SM == SM_UE8M0)
      scb[jj] = __uint_as_float(__float_as_uint(scp[(HALF * G_HT + jj) * 16]) >> ((kb & 3) * 8));
    else if constexpr (SM == SM_EPILOGUE)
      scb[jj] = __int_as_float(in_vgpr(127));  // (a constant, too, is put into its register where every lane is active)
    else
      scb[jj] = scp[(HALF * G_HT + jj) * 16] * sbv;
  }
}

// The promotion of the last MFMA of a compute phase is left to the start of the wave's next memory phase (the other
// group's MFMAs already own the pipe by then), so a compute phase does not end on a wait for its own last result.
struct Pending {
  v4f part;
  float scale;
};

template <int HALF>
__device__ __forceinline__ void retire(const Pending& pd, float (&acc)[G_NT][G_MT][4]) {
#pragma unroll
  for (int v = 0; v < 4; ++v)
    acc[G_NT - 1][HALF * G_HT + G_HT - 1][v] = fmaf(pd.part[v], pd.scale, acc[G_NT - 1][HALF * G_HT + G_HT - 1][v]);
}

// Compute phase: 16 steps of {MFMA of tile t, promotion FMAs of tile t - 2}.  The FMAs lag by two MFMAs (three result
// buffers), so they never wait for a result that is still in the pipe (measured 3.5 % faster than a lag of one).
template <int HALF>
__device__ __forceinline__ void compute(const Frag (&w)[G_NT], const Frag (&tok)[G_HT], const float (&scb)[G_HT],
                                        float (&acc)[G_NT][G_MT][4], Pending& pd) {
  constexpr int STEPS = G_HT * G_NT;
  v4f part[3];
#pragma unroll
  for (int t = 0; t < STEPS + 1; ++t) {
    if (t < STEPS) {
      const int jj = t >> 2, i = t & 3;
      part[t % 3] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(as_v8i(w[i]), as_v8i(tok[jj]), v4f{0.f, 0.f, 0.f, 0.f},
                                                                     0, 0, 0, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);  // the MFMA goes first; the FMAs run in its shadow
    }
    if (t > 1) {
      const int pj = (t - 2) >> 2, pi = (t - 2) & 3;
#pragma unroll
      for (int v = 0; v < 4; ++v)
        acc[pi][HALF * G_HT + pj][v] = fmaf(part[(t - 2) % 3][v], scb[pj], acc[pi][HALF * G_HT + pj][v]);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  pd.part = part[(STEPS - 1) % 3];
  pd.scale = scb[G_HT - 1];
}

// Compute phase with power-of-two scales on both sides: the MFMA applies them itself (scale operands: byte 0 of each
// lane's register; lane l supplies the scale of operand row l % 16 for K sub-block l / 16 - here one value per row), so
// the products go straight into the accumulators and no vector arithmetic is left in the phase.
template <int HALF>
__device__ __forceinline__ void compute_ue8m0(const Frag (&w)[G_NT], const Frag (&tok)[G_HT], const float (&scb)[G_HT],
                                              int w_scale, float (&acc)[G_NT][G_MT][4]) {
#pragma unroll
  for (int jj = 0; jj < G_HT; ++jj)
#pragma unroll
    for (int i = 0; i < G_NT; ++i) {
      float* a = acc[i][HALF * G_HT + jj];
      const v4f r = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(as_v8i(w[i]), as_v8i(tok[jj]), v4f{a[0], a[1], a[2], a[3]}, 0,
                                                                     0, 0, w_scale, 0, (int)__float_as_uint(scb[jj]));
      a[0] = r[0], a[1] = r[1], a[2] = r[2], a[3] = r[3];
    }
  __builtin_amdgcn_sched_barrier(0);
}

// r[v] = row_scale[m] * (col_scale[n + v] * r[v]) + bias[n + v], each step rounded (the order of fp8_scaled_mm's epilogue,
// sgl-kernel/csrc/gemm/fp8_gemm_kernel.cu:529-547); channels at or past N repeat the last one and are never stored.
__device__ __forceinline__ void row_col_epilogue(const GemmParams& p, int m, int n, float* r) {
  const float rs = p.row_scale[min(m, p.M - 1)];
  const uint16_t* b = reinterpret_cast<const uint16_t*>(p.bias);
  float cs[4], bv[4] = {0.f, 0.f, 0.f, 0.f};
  if (n + 4 <= p.N && (reinterpret_cast<uintptr_t>(p.col_scale + n) & 15) == 0 &&
      (p.bias == nullptr || (reinterpret_cast<uintptr_t>(b + n) & 7) == 0)) {
    // one 16-byte and one 8-byte load instead of eight scattered ones
    const v4f c = *reinterpret_cast<const v4f*>(p.col_scale + n);
    cs[0] = c[0], cs[1] = c[1], cs[2] = c[2], cs[3] = c[3];
    if (p.bias) {
      const u32x2 hb = *reinterpret_cast<const u32x2*>(b + n);
      const uint32_t h[4] = {hb.x & 0xffffu, hb.x >> 16, hb.y & 0xffffu, hb.y >> 16};
#pragma unroll
      for (int v = 0; v < 4; ++v) bv[v] = (p.out_dtype == MI355_BF16) ? bf16_bits_to_f32(h[v]) : f16_bits_to_f32(h[v]);
    }
  } else {
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int nn = min(n + v, p.N - 1);
      cs[v] = p.col_scale[nn];
      if (p.bias) bv[v] = (p.out_dtype == MI355_BF16) ? bf16_bits_to_f32(b[nn]) : f16_bits_to_f32(b[nn]);
    }
  }
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const float t = mul_rn(rs, mul_rn(cs[v], r[v]));
    r[v] = p.bias ? add_rn(t, bv[v]) : t;
  }
}

// SM, where the scales are applied:
//   SM_BLOCK_F32  fp32 scales per K block, by promotion FMAs (the blockwise GEMM of the reference);
//   SM_UE8M0      p.sa / p.sb point to packed exponent words (int32): token word (m, kw) at sa[kw * sa_sk + m], channel word
//                 (n, kw) at sb[kw * sb_sk + n * sb_sn], byte kb & 3 of word kb >> 2 belongs to K block kb; the MFMA applies them;
//   SM_EPILOGUE   one scale per token (p.row_scale) and per channel (p.col_scale), applied once, after the K loop, as
//                 row_scale * (col_scale * acc) + bias; the K loop accumulates in the MFMA with unit scales.
// NOLOAD (a measurement aid, never the product): K blocks 0 and 1 and the token scales of blocks 0..3 are fetched once and
// every later K block multiplies those again, so the loop is the product's instruction stream on the product's operand
// values minus its global loads; what it leaves out is what the loads cost.
// One 256 x 256 output tile at (m0, n0) by the whole workgroup.
template <bool KFULL, int SM, bool NOLOAD = false>
__device__ __forceinline__ void pp_tile(const GemmParams& p, const int m0, const int n0) {
  constexpr bool UE8M0 = SM == SM_UE8M0;
  constexpr bool HW_SCALE = SM != SM_BLOCK_F32;  // scale operands of the MFMA instead of promotion FMAs
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = wave >> 2;  // 0: starts computing first; 1: one phase behind.  Also the wave's token half of the tile.
  const int wave_n = wave & 3;
  const int l16 = lane & 15, q = lane >> 4;

  const int nkb = p.kb_total;

  PpState s;
  s.K = p.K;
  s.wave = wave;
  s.kb_last = nkb - 1;
  s.a_base = p.a;
  s.b_base = p.b;
  {
    // lane l of a wave lands in row l / 8, physical chunk l % 8 of the 8 rows one load fills; it fetches the logical
    // chunk that belongs there under the (row & 7) swizzle
    const int lrow = lane >> 3;
    s.chunk_byte = ((lane & 7) ^ lrow) * 16;
#pragma unroll
    for (int i = 0; i < G_LOADS; ++i) {
      const int row = i * 64 + wave * 8 + lrow;
      if (row < G_BM)
        s.goff[i] = (uint32_t)((int64_t)min(m0 + row, p.M - 1) * p.lda + s.chunk_byte);
      else
        s.goff[i] = (uint32_t)((int64_t)min(n0 + row - G_BM, p.N - 1) * p.ldb + s.chunk_byte);
    }
    const int trow = grp * G_WM + l16, crow = G_BM + wave_n * G_WN + l16;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      s.tok_off[h] = trow * KSTEP + (((q + 4 * h) ^ (trow & 7)) << 4);
      s.ch_off[h] = crow * KSTEP + (((q + 4 * h) ^ (crow & 7)) << 4);
    }
    s.sc_off = (grp * G_WM + l16) * 4;
  }
  s.sa_base = p.sa;
  s.sa_off = (uint32_t)min(m0 + wave * 32 + (lane & 7) * 4, (p.M - 1) & ~3) * 4u;  // quads past M refetch the last one
  s.sa_sk = p.sa_sk;
  s.sb_ptr = (cfloat_ptr)(p.sb + (int64_t)__builtin_amdgcn_readfirstlane(UE8M0 ? min(n0 + wave_n * G_WN, p.N - 1)
                                                                                  : min(n0 + wave_n * G_WN, p.N - 1) / 128) *
                                     p.sb_sn);
  s.sb_sk = p.sb_sk;

  float acc[G_NT][G_MT][4];
#pragma unroll
  for (int i = 0; i < G_NT; ++i)
#pragma unroll
    for (int j = 0; j < G_MT; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.f;

  Frag w[G_NT], tok[G_HT];
  float scb[G_HT];
  Pending pd;
  pd.part = v4f{0.f, 0.f, 0.f, 0.f};
  pd.scale = 0.f;

  // ---- prologue: all of block 0 and set A of block 1
  issue_set_a<KFULL, UE8M0>(s, g_stage0, 0);
  issue_set_b<KFULL>(s, g_stage0, 0);
  issue_set_a<KFULL, UE8M0>(s, g_stage1, 1);
  float sb_cur = s.sb_ptr[0];
  if constexpr (NOLOAD) {
    issue_set_b<KFULL>(s, g_stage1, 1);
    issue_scales<UE8M0>(s, 2);
    issue_scales<UE8M0>(s, 3);
    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
  } else {
    asm volatile("s_waitcnt vmcnt(7)\n\ts_barrier" ::: "memory");  // block 0 is in LDS (set A of block 1 may be in flight)
  }
  if (grp == 1) compute_end();  // group 1 runs one phase behind group 0

  // One K block: M0, C0, M1, C1.  `cur` holds block kb; `nxt` takes set B of block kb + 1, `cur` set A of block kb + 2.
  auto k_block = [&](uint8_t* cur, uint8_t* nxt, int kb, float sbv) {
    const float* sc_cur = g_scale + (kb & 3) * G_BM;
    // the weight block's exponent byte, in byte 0 of a register (for SM_UE8M0 sbv carries the packed word as bits)
    const int w_scale = HW_SCALE ? in_vgpr(UE8M0 ? (int)(__float_as_uint(sbv) >> ((kb & 3) * 8)) : 127) : 127;
    if constexpr (!HW_SCALE) retire<1>(pd, acc);  // last tile of the previous block (adds zero the first time)
    read_operands<0, SM>(s, cur, sc_cur, sbv, kb, w, tok, scb);
    if constexpr (!NOLOAD) issue_set_b<KFULL>(s, nxt, kb + 1);
    memory_end();
    if constexpr (HW_SCALE) compute_ue8m0<0>(w, tok, scb, w_scale, acc);
    else compute<0>(w, tok, scb, acc, pd);
    compute_end();
    if constexpr (!HW_SCALE) retire<0>(pd, acc);
    read_operands<1, SM>(s, cur, sc_cur, sbv, kb, w, tok, scb);
    if constexpr (!NOLOAD) issue_set_a<KFULL, UE8M0>(s, cur, kb + 2);
    memory_end();
    if constexpr (HW_SCALE) compute_ue8m0<1>(w, tok, scb, w_scale, acc);
    else compute<1>(w, tok, scb, acc, pd);
    compute_end();
  };

  int kb = 0;
  for (; kb + 1 < nkb; kb += 2) {
    const float sb_1 = s.sb_ptr[(int64_t)(UE8M0 ? (kb + 1) >> 2 : kb + 1) * s.sb_sk];
    const float sb_2 = s.sb_ptr[(int64_t)(UE8M0 ? min(kb + 2, nkb - 1) >> 2 : min(kb + 2, nkb - 1)) * s.sb_sk];
    k_block(g_stage0, g_stage1, kb, sb_cur);
    k_block(g_stage1, g_stage0, kb + 1, sb_1);
    sb_cur = sb_2;
  }
  if (kb < nkb) k_block(g_stage0, g_stage1, kb, sb_cur);
  if constexpr (!HW_SCALE) retire<1>(pd, acc);
  if (grp == 0) compute_end();  // as many barriers as group 1
  // the last requests refetch the last block into rows nobody reads any more: they must not outlive the workgroup's LDS
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  // ---- epilogue: lane holds channels n .. n+3 of token m
  if (out_tile_ok(p.out, p.ldo, p.out_dtype, n0, p.N)) {
    asm volatile("s_barrier" ::: "memory");  // every wave's stray loads have landed: the stages are free
#pragma unroll
    for (int j = 0; j < G_MT; ++j)
#pragma unroll
      for (int i = 0; i < G_NT; ++i) {
        if constexpr (SM == SM_EPILOGUE) row_col_epilogue(p, m0 + grp * G_WM + j * 16 + l16, n0 + wave_n * G_WN + i * 16 + 4 * q, acc[i][j]);
        else fp8_channel_epilogue(p, n0 + wave_n * G_WN + i * 16 + 4 * q, acc[i][j]);
        out_tile_put4(g_stages, grp * G_WM + j * 16 + l16, wave_n * G_WN + i * 16 + 4 * q, p.out_dtype, acc[i][j]);
      }
    __syncthreads();
    out_tile_store(g_stages, p.out, p.ldo, m0, n0, p.M);
    return;
  }
  const bool vec_ok = ((p.ldo & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
#pragma unroll
  for (int j = 0; j < G_MT; ++j) {
    const int m = m0 + grp * G_WM + j * 16 + l16;
    if (m >= p.M) continue;
#pragma unroll
    for (int i = 0; i < G_NT; ++i) {
      const int n = n0 + wave_n * G_WN + i * 16 + 4 * q;
      if (n >= p.N) continue;
      if constexpr (SM == SM_EPILOGUE) row_col_epilogue(p, m, n, acc[i][j]);
      else fp8_channel_epilogue(p, n, acc[i][j]);
      store_out4(p.out, p.out_dtype, (int64_t)m * p.ldo + n, acc[i][j], min(4, p.N - n), vec_ok);
    }
  }
}

template <bool KFULL, int SM, bool NOLOAD = false>
__global__ __launch_bounds__(G_THREADS) void fp8_gemm_pp_kernel(const GemmParams p) {
  const TileCoord tc = tile_of_block(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n);
  pp_tile<KFULL, SM, NOLOAD>(p, tc.tile_m * G_BM, tc.tile_n * G_BN);
}

// Grouped problems (see GroupedParams): the workgroup's token tile comes from the table the plan kernel wrote, the
// operand bases move to that tile's expert.  Workgroup order as in fp8_grouped_dma3_kernel.
__global__ __launch_bounds__(G_THREADS) void fp8_grouped_pp_kernel(const GroupedParams gp) {
  GemmParams p;
  int m0, tile_n;
  if (!grouped_tile_of_block(gp, p, m0, tile_n)) return;  // the whole workgroup leaves before any barrier
  pp_tile<true, SM_BLOCK_F32>(p, m0, tile_n * G_BN);
}

}  // namespace

int launch_fp8_grouped_pp(GroupedParams& gp, hipStream_t stream, const char* what) {
  gp.g.tiles_n = (gp.g.N + G_BN - 1) / G_BN;
  gp.g.splits = 1, gp.g.kb_per_split = gp.g.kb_total;
  const dim3 grid((unsigned)(gp.max_tiles_m * gp.g.tiles_n));
  hipLaunchKernelGGL(fp8_grouped_pp_kernel, grid, dim3(G_THREADS), 0, stream, gp);
  return check_launch(what);
}

// Needs 16-byte aligned rows, row offsets below 4 GiB and conforming token scales (fp8_scales_conform).
int launch_fp8_pp(GemmParams& p, hipStream_t stream, const char* what) {
  p.tiles_m = (p.M + G_BM - 1) / G_BM;
  p.tiles_n = (p.N + G_BN - 1) / G_BN;
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n));
  if (p.K % KSTEP == 0)
    hipLaunchKernelGGL((fp8_gemm_pp_kernel<true, SM_BLOCK_F32>), grid, dim3(G_THREADS), 0, stream, p);
  else
    hipLaunchKernelGGL((fp8_gemm_pp_kernel<false, SM_BLOCK_F32>), grid, dim3(G_THREADS), 0, stream, p);
  return check_launch(what);
}

// The K loop of launch_fp8_pp without its global loads (NOLOAD above): a measurement aid.  K % 128 == 0, K >= 512.
int launch_fp8_pp_noload(GemmParams& p, hipStream_t stream, const char* what) {
  p.tiles_m = (p.M + G_BM - 1) / G_BM;
  p.tiles_n = (p.N + G_BN - 1) / G_BN;
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n));
  hipLaunchKernelGGL((fp8_gemm_pp_kernel<true, SM_BLOCK_F32, true>), grid, dim3(G_THREADS), 0, stream, p);
  return check_launch(what);
}

// The same kernel with packed power-of-two scales on both operands (see fp8_gemm_pp_kernel).  Needs K % 128 == 0, token
// words M-major with a pitch that is a multiple of four words and a 16-byte aligned base.
int launch_fp8_pp_ue8m0(GemmParams& p, hipStream_t stream, const char* what) {
  p.tiles_m = (p.M + G_BM - 1) / G_BM;
  p.tiles_n = (p.N + G_BN - 1) / G_BN;
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n));
  hipLaunchKernelGGL((fp8_gemm_pp_kernel<true, SM_UE8M0>), grid, dim3(G_THREADS), 0, stream, p);
  return check_launch(what);
}


// Per-token x per-channel scales applied in the epilogue (p.row_scale [M], p.col_scale [N], optional p.bias); the K loop
// runs without any scale arithmetic.  p.sa must point to at least 4 * M readable, 16-byte aligned bytes (the scale-load
// slots of the schedule still fetch, nobody reads what they bring) and p.sb to one readable float.  K % 128 == 0.
int launch_fp8_pp_rowcol(GemmParams& p, hipStream_t stream, const char* what) {
  p.tiles_m = (p.M + G_BM - 1) / G_BM;
  p.tiles_n = (p.N + G_BN - 1) / G_BN;
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n));
  hipLaunchKernelGGL((fp8_gemm_pp_kernel<true, SM_EPILOGUE>), grid, dim3(G_THREADS), 0, stream, p);
  return check_launch(what);
}

}  // namespace mi355
