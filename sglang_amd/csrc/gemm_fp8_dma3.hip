// Blockwise-scaled FP8 GEMM for gfx950 with short token tiles: (64 or 128) x (256, 192 or 128) macro tile, 8 waves (two per SIMD),
// THREE LDS stages (four for 64 x 192 and 128 x 128 tiles, six for 64 x 128 tiles when a workgroup has a CU to itself); the 128-token
// tiles run with two extra loader waves (dma3_tile_lw).
//
// For 16 < M <= 1024 a linear layer is between weight streaming and MFMA-bound; prefill shapes with few output channels
// (M = 4096, N = 576 or 1536) do not give 256 x 256 tiles enough workgroups.  Both take this kernel.  The tile is short in the token dimension
// (64 or 128 tokens) and wide in channels (256; 192 and 128 where those fill the chip better: 36864 channels are 144 tiles
// of 256 but 192 of 192, 1536 channels x 4096 tokens are exactly 256 tiles of 128 x 192), so a stage of LDS is
// (BM + BN) x 128 B <= 48 KB and three stages fit in the CU's 160 KB.  With three stages the direct-to-LDS loads of K block k+2 are issued while block k is multiplied and
// only have to land before block k+2 is multiplied, two barriers later: the wait that precedes the barrier at the end of
// iteration k covers block k+1 only.  The compiler cannot express that (its wait before a barrier covers every load it
// knows about), so inside the loop the loads, the wait and the barrier are written as instructions:
//   * every iteration issues exactly LOADS + 1 loads per wave (tile rows plus the token scales), always, even past the
//     end of K (they refetch the last block into a stage nobody reads), so "block k+1 has landed" is the constant
//     s_waitcnt vmcnt(LOADS + 1): everything but the youngest LOADS + 1 loads;
//   * nothing else in the loop counts in vmcnt (weight-block scales come by scalar loads);
//   * the barrier is a bare s_barrier: LDS written by the loads is complete when vmcnt says so, and a stage is
//     overwritten only after the barrier that follows its last read.
// Operand roles, swizzle, chunk mapping and promotion FMA are those of gemm_w8a8.hip; a step is {MFMA of tile t, FMAs of
// tile t-1}.  Optional split along K (partials to the workspace, ordered reduce afterwards).
// Requires K % 128 == 0, 16-byte aligned rows, row offsets below 4 GiB, and token scales laid out M-major with a pitch that is
// a multiple of four floats (fp8_scales_conform; the dispatcher re-lays other layouts out into the workspace first).
#include "gemm_common.h"

namespace mi355 {
namespace {

constexpr int T_THREADS = 512;
constexpr int T_BN = 256;  // widest channel tile (sizes the LDS stages); the kernels take BN = 128 or 256

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;
typedef const __attribute__((address_space(3))) uint8_t* lds_cptr;
typedef const __attribute__((address_space(4))) float* cfloat_ptr;

struct Frag {
  u32x4 lo, hi;
};
__device__ __forceinline__ v8i as_v8i(const Frag& f) {
  return v8i{(int)f.lo.x, (int)f.lo.y, (int)f.lo.z, (int)f.lo.w, (int)f.hi.x, (int)f.hi.y, (int)f.hi.z, (int)f.hi.w};
}
__device__ __forceinline__ u32x4 lds16(lds_cptr p, int imm) {
  return *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(p + imm);
}

template <int BM, int BN>
struct Dma3State {
  static constexpr int LOADS = (BM + BN) / 64;  // tile loads per wave and stage (a wave fills 8 rows per load)
  const uint8_t* a_base;
  const uint8_t* b_base;
  uint32_t goff[LOADS];   // lane's byte offset from the matrix base (rows clamped); first BM/64 loads are token rows
  const float* sa_base;   // token scales, M-major: element (m, kb) at sa_base[kb * sa_sk + m]
  uint32_t sa_off;        // byte offset of the four scales this lane fetches (first BM / 32 lanes), clamped to the last valid quad
  // Weight-block scale rows.  A wave's channels are BN / 4 consecutive ones inside one 128-channel block, except for
  // BN = 192, where 48 consecutive channels could straddle two blocks: there the wave's tile i is channels
  // 64 i + 16 wave .. + 15 of the tile, so that tile i of every wave lies in the block of channel n0 + 64 i.
  static constexpr bool INTERLEAVED = BN == 192;
  static constexpr int SB = INTERLEAVED ? BN / 64 : 1;
  static constexpr int W_STRIDE = INTERLEAVED ? 64 * 128 : 16 * 128;  // bytes between a wave's consecutive channel tiles in a stage
  cfloat_ptr sb_ptr[SB];  // &sb[nb, 0] of the wave's (tile's) 128-channel block
  int64_t sa_sk, sb_sk;
  int wave, kb_last;
  uint32_t tok_off[2], ch_off[2], sc_off;
};

// Load number i (< LOADS: tile rows; == LOADS: token scales) of K block kb, written as instructions.
// The statements write m0; it cannot be listed as a clobber (the compiler reserves the register and rejects the entry), and
// no compiler-managed use of m0 lies between them and the next statement that sets it.
template <int BM, int BN, bool UE8M0 = false>
__device__ __forceinline__ void issue_one(const Dma3State<BM, BN>& s, int i, uint8_t* stage, float* scale, int kb) {
  constexpr int LOADS = Dma3State<BM, BN>::LOADS;
  kb = min(kb, s.kb_last);
  if (i < LOADS) {
    const uint8_t* base = (i < BM / 64 ? s.a_base : s.b_base) + (uint64_t)kb * KSTEP;  // wave-uniform
    asm volatile("" : "+s"(base));
    const uint32_t lds_addr = (uint32_t)(uintptr_t)(lptr_t)(stage + (i * 64 + s.wave * 8) * KSTEP);
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(s.goff[i]), "s"(base), "s"(lds_addr) : "memory");
  } else {
    // the wave's BM / 8 token scales: BM / 32 lanes fetch 16 bytes each (a 4-byte-per-lane load in this stream costs far
    // more than its size: measured 1.5x on the whole large-M kernel).  exec is narrowed and restored inside the statement.
    // fp32 scales: one row of floats per K block; packed exponents: one row of 32-bit words per four K blocks, fetched
    // again for each of the four (the load count per K block stays constant)
    const float* sbase = s.sa_base + (int64_t)(UE8M0 ? kb >> 2 : kb) * s.sa_sk;  // wave-uniform
    asm volatile("" : "+s"(sbase));
    const uint32_t lds_addr = (uint32_t)(uintptr_t)(lptr_t)(scale + s.wave * (BM / 8));
    uint64_t saved;
    if constexpr (BM == 128)
      asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, 0xf\n\ts_mov_b32 m0, %3\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b64 exec, %0"
                   : "=&s"(saved) : "v"(s.sa_off), "s"(sbase), "s"(lds_addr) : "memory");
    else
      asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, 0x3\n\ts_mov_b32 m0, %3\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b64 exec, %0"
                   : "=&s"(saved) : "v"(s.sa_off), "s"(sbase), "s"(lds_addr) : "memory");
  }
}

// One K block out of `cur`; the loads of block kb_next go out over the first LOADS + 1 steps into `nxt`.
// UE8M0: the scale stage holds the tokens' packed exponent words and sbv the weight blocks' (as bits); the byte of block
// `kb` goes to the MFMA, which applies both scales and accumulates in place: no promotion FMAs.
// ISSUE: 1 = the wave issues its share of every load of block kb_next (tile rows and token scales), 2 = of the weight rows
// only (a producer wave writes the tokens), 0 = none (loader waves do).
template <int BM, int BN, bool UE8M0 = false, int ISSUE = 1>
__device__ __forceinline__ void k_block(const Dma3State<BM, BN>& s, const uint8_t* cur, const float* sc_cur,
                                        const float (&sbv)[Dma3State<BM, BN>::SB], float (&acc)[BN / 64][BM / 32][4], uint8_t* nxt,
                                        float* sc_nxt, int kb_next, int kb = 0) {
  constexpr int MT = BM / 32, T_NT = BN / 64, LOADS = Dma3State<BM, BN>::LOADS;  // a wave owns BN / 4 channels = T_NT tiles of 16
  constexpr int SB = Dma3State<BM, BN>::SB, W_STRIDE = Dma3State<BM, BN>::W_STRIDE;
  static_assert(LOADS + 1 <= MT * T_NT, "one load per step");
  Frag w[T_NT], tokb[2];
  float scb[2][SB];
  const lds_cptr ch0 = (lds_cptr)cur + s.ch_off[0], ch1 = (lds_cptr)cur + s.ch_off[1];
  const lds_cptr tk0 = (lds_cptr)cur + s.tok_off[0], tk1 = (lds_cptr)cur + s.tok_off[1];
  w[0].lo = lds16(ch0, 0);
  w[0].hi = lds16(ch1, 0);
  tokb[0].lo = lds16(tk0, 0);
  tokb[0].hi = lds16(tk1, 0);
  const float* scp = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(sc_cur) + s.sc_off);
  const int shift = (kb & 3) * 8;
  int w_exp[SB];  // UE8M0: the weight blocks' exponent bytes of this K block, in byte 0
#pragma unroll
  for (int b = 0; b < SB; ++b) {
    if constexpr (UE8M0) {
      w_exp[b] = in_vgpr((int)(__float_as_uint(sbv[b]) >> shift));
      scb[0][b] = __uint_as_float(__float_as_uint(scp[0]) >> shift);
    } else {
      w_exp[b] = 0;
      scb[0][b] = scp[0] * sbv[b];
    }
  }
  __builtin_amdgcn_sched_barrier(0);

  v4f part[2];
#pragma unroll
  for (int t = 0; t < MT * T_NT; ++t) {
    const int j = t / T_NT, i = t % T_NT;
    if constexpr (UE8M0) {
      float* a = acc[i][j];
      const v4f r = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(as_v8i(w[i]), as_v8i(tokb[j & 1]), v4f{a[0], a[1], a[2], a[3]}, 0, 0, 0,
                                                                     w_exp[SB > 1 ? i : 0], 0, (int)__float_as_uint(scb[j & 1][0]));
      a[0] = r[0], a[1] = r[1], a[2] = r[2], a[3] = r[3];
    } else {
      part[t & 1] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(as_v8i(w[i]), as_v8i(tokb[j & 1]),
                                                                     v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);  // the MFMA goes first; the rest of the step runs in its shadow
    if (!UE8M0 && t > 0) {
      const int pj = (t - 1) / T_NT, pi = (t - 1) % T_NT;
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[pi][pj][v] = fmaf(part[(t - 1) & 1][v], scb[pj & 1][SB > 1 ? pi : 0], acc[pi][pj][v]);
    }
    if (t + 1 < T_NT) {  // remaining weight fragments, one per step
      w[t + 1].lo = lds16(ch0, (t + 1) * W_STRIDE);
      w[t + 1].hi = lds16(ch1, (t + 1) * W_STRIDE);
    }
    if (i == 0 && j + 1 < MT) {  // next token tile
      tokb[(j + 1) & 1].lo = lds16(tk0, (j + 1) * 2048);
      tokb[(j + 1) & 1].hi = lds16(tk1, (j + 1) * 2048);
    }
    if (i == 1 && j + 1 < MT) {
#pragma unroll
      for (int b = 0; b < SB; ++b) {
        if constexpr (UE8M0) scb[(j + 1) & 1][b] = __uint_as_float(__float_as_uint(scp[(j + 1) * 16]) >> shift);
        else scb[(j + 1) & 1][b] = scp[(j + 1) * 16] * sbv[b];
      }
    }
    if (ISSUE == 1 && t <= LOADS) issue_one<BM, BN, UE8M0>(s, t, nxt, sc_nxt, kb_next);
    if (ISSUE == 2 && t >= BM / 64 && t < LOADS) issue_one<BM, BN, UE8M0>(s, t, nxt, sc_nxt, kb_next);
    __builtin_amdgcn_sched_barrier(0);
  }
  if constexpr (!UE8M0) {
    constexpr int t = MT * T_NT - 1;
    constexpr int pj = t / T_NT, pi = t % T_NT;
#pragma unroll
    for (int v = 0; v < 4; ++v) acc[pi][pj][v] = fmaf(part[t & 1][v], scb[pj & 1][SB > 1 ? pi : 0], acc[pi][pj][v]);
  }
}

// Everything but the YOUNGER youngest loads has landed; then the workgroup barrier.  Instructions, see the file comment.
template <int YOUNGER>
__device__ __forceinline__ void wait_and_barrier() {
  static_assert(YOUNGER >= 4 && YOUNGER <= 28, "(stages - 2) x (LOADS + 1), LOADS + 1 = (BM + BN) / 64 + 1");
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(YOUNGER) : "memory");
}

// Epilogue of a compute wave: the lane holds channels n .. n+3 of token m for each of its MFMA tiles; raw partial sums to the
// workspace (SPLIT) or channel epilogue, conversion and store.
template <int BM, bool SPLIT, int BN>
__device__ __forceinline__ void store_tile(const GemmParams& p, float (&acc)[BN / 64][BM / 32][4], int m0, int n0, int split, int wave_m,
                                           int wave_n, int l16, int q) {
  constexpr int WM = BM / 2, MT = WM / 16, T_WN = BN / 4, T_NT = T_WN / 16;
  constexpr bool INTERLEAVED = Dma3State<BM, BN>::INTERLEAVED;
  const bool vec_ok = ((p.ldo & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    const int m = m0 + wave_m * WM + j * 16 + l16;
    if (m >= p.M) continue;
#pragma unroll
    for (int i = 0; i < T_NT; ++i) {
      const int n = n0 + (INTERLEAVED ? i * 64 + wave_n * 16 : wave_n * T_WN + i * 16) + 4 * q;
      if (n >= p.N) continue;
      const int nvalid = min(4, p.N - n);
      if constexpr (SPLIT) {
        float* wsp = reinterpret_cast<float*>(p.ws) + ((int64_t)split * p.M + m) * p.N + n;
#pragma unroll
        for (int v = 0; v < 4; ++v)
          if (v < nvalid) wsp[v] = acc[i][j][v];
      } else {
        fp8_channel_epilogue(p, n, acc[i][j]);
        store_out4(p.out, p.out_dtype, (int64_t)m * p.ldo + n, acc[i][j], nvalid, vec_ok);
      }
    }
  }
}

// One BM x 256 output tile at (m0, n0), K blocks of split `split`, by the whole workgroup.
// UE8M0: p.sa / p.sb point to packed exponent words (int32): token word (m, kw) at sa[kw * sa_sk + m], channel word (n, kw)
// at sb[kw * sb_sk + n * sb_sn], byte kb & 3 of word kb >> 2 belongs to K block kb; the MFMA applies them.
// S: LDS stages (S - 1 K blocks in flight).  Three everywhere; more where the tile is small enough for them to fit and the
// launch has at most one workgroup per CU, so that nothing else would use the LDS.
template <int BM, bool SPLIT, int BN = T_BN, bool UE8M0 = false, int S = 3>
__device__ __forceinline__ void dma3_tile(const GemmParams& p, int m0, int n0, int split) {
  static_assert(BN == 128 || BN == 192 || BN == 256, "channel tile");
  static_assert(S >= 3 && S * ((BM + BN) * KSTEP + BM * 4) <= 160 * 1024, "the stages must fit the CU's LDS");
  constexpr int WM = BM / 2, MT = WM / 16, T_WN = BN / 4, T_NT = T_WN / 16, LOADS = Dma3State<BM, BN>::LOADS;
  constexpr bool INTERLEAVED = Dma3State<BM, BN>::INTERLEAVED;
  constexpr int SB = Dma3State<BM, BN>::SB;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave >> 2, wave_n = wave & 3;
  const int l16 = lane & 15, q = lane >> 4;

  const int kb_begin = split * p.kb_per_split;
  const int kb_end = min(p.kb_total, kb_begin + p.kb_per_split);
  const int nkb = kb_end - kb_begin;

  Dma3State<BM, BN> s;
  s.wave = wave;
  s.kb_last = kb_end - 1;
  s.a_base = p.a;
  s.b_base = p.b;
  {
    const int lrow = lane >> 3;
    const int chunk_byte = ((lane & 7) ^ lrow) * 16;  // lane fetches the chunk that lands swizzled by (row & 7)
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int row = i * 64 + wave * 8 + lrow;
      if (row < BM)
        s.goff[i] = (uint32_t)((int64_t)min(m0 + row, p.M - 1) * p.lda + chunk_byte);
      else
        s.goff[i] = (uint32_t)((int64_t)min(n0 + row - BM, p.N - 1) * p.ldb + chunk_byte);
    }
    const int trow = wave_m * WM + l16, crow = BM + wave_n * (INTERLEAVED ? 16 : T_WN) + l16;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      s.tok_off[h] = trow * KSTEP + (((q + 4 * h) ^ (trow & 7)) << 4);
      s.ch_off[h] = crow * KSTEP + (((q + 4 * h) ^ (crow & 7)) << 4);
    }
    s.sc_off = (wave_m * WM + l16) * 4;
  }
  // every wave fetches BM / 8 token scales per K block, four per lane; quads past M refetch the last valid one
  s.sa_base = p.sa;
  s.sa_off = (uint32_t)min(m0 + wave * (BM / 8) + (lane & (BM / 32 - 1)) * 4, (p.M - 1) & ~3) * 4u;
  s.sa_sk = p.sa_sk;
#pragma unroll
  for (int b = 0; b < SB; ++b) {
    const int first = INTERLEAVED ? n0 + 64 * b : n0 + wave_n * T_WN;  // first channel of the wave's tile(s) with this scale
    s.sb_ptr[b] = (cfloat_ptr)(p.sb + (int64_t)__builtin_amdgcn_readfirstlane(UE8M0 ? min(first, p.N - 1) : min(first, p.N - 1) / 128) * p.sb_sn);
  }
  s.sb_sk = p.sb_sk;

  // the stages: tiles (rows 0..BM-1 tokens, BM.. channels) and the tile's BM token scales, sized per tile shape: three
  // stages of a 64 x 128 tile take 73.5 KB, so two such workgroups share a CU's 160 KB
  __shared__ __attribute__((aligned(1024))) uint8_t t_stage[S][(BM + BN) * KSTEP];
  __shared__ __attribute__((aligned(256))) float t_scale[S][BM];
  // PAIRED (six stages): one barrier per TWO K blocks (1-4 % over a barrier per block: K=7168 -> N=576 at M=2048 27.0 ->
  // 26.3 us, K=7168 -> N=4096 at M=512 25.2 -> 24.3, K=7168 -> N=1536 at M=128 16.9 -> 16.5; never slower).  Iteration k requests block k + S - 2 into the stage that iteration
  // k - 2 read, so the barrier after every odd iteration separates all reads of a stage from the next loads into it, and the
  // wait in front of it covers the two blocks of the next pair: the S - 4 blocks requested after them may be in flight.
  constexpr bool PAIRED = S == 6;
  constexpr int AHEAD = PAIRED ? S - 2 : S - 1;                                 // blocks requested ahead of the one multiplied
  constexpr int YOUNGER = (PAIRED ? S - 4 : S - 2) * (LOADS + 1);              // loads that may be in flight at a barrier

  float acc[T_NT][MT][4];
#pragma unroll
  for (int i = 0; i < T_NT; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.f;

  // ---- prologue: blocks 0 .. AHEAD-1 (clamped) into stages 0 .. AHEAD-1
#pragma unroll
  for (int b = 0; b < AHEAD; ++b)
#pragma unroll
    for (int i = 0; i <= LOADS; ++i) issue_one<BM, BN, UE8M0>(s, i, t_stage[b], t_scale[b], kb_begin + b);
  wait_and_barrier<YOUNGER>();  // block 0 (PAIRED: and block 1) has landed everywhere

  // ---- S blocks per trip over the S stages; iteration k multiplies block k and requests block k + AHEAD into the stage
  //      that iteration k - 1 (PAIRED: k - 2) read
  auto sb_of = [&](int kb, float (&v)[SB]) {
#pragma unroll
    for (int b = 0; b < SB; ++b) v[b] = s.sb_ptr[b][(int64_t)(UE8M0 ? kb >> 2 : kb) * s.sb_sk];
  };
  int k = 0;
  for (; k + S - 1 < nkb; k += S) {
    float sbv[S][SB];
#pragma unroll
    for (int u = 0; u < S; ++u) sb_of(kb_begin + k + u, sbv[u]);
#pragma unroll
    for (int u = 0; u < S; ++u) {
      k_block<BM, BN, UE8M0>(s, t_stage[u], t_scale[u], sbv[u], acc, t_stage[(u + AHEAD) % S], t_scale[(u + AHEAD) % S],
                             kb_begin + k + u + AHEAD, kb_begin + k + u);
      if (!PAIRED || (u & 1)) wait_and_barrier<YOUNGER>();
    }
  }
#pragma unroll
  for (int u = 0; u < S - 1; ++u) {  // up to S - 1 blocks left, in stages 0 ..
    if (k + u < nkb) {
      float sbl[SB];
      sb_of(kb_begin + k + u, sbl);
      k_block<BM, BN, UE8M0>(s, t_stage[u], t_scale[u], sbl, acc, t_stage[(u + AHEAD) % S], t_scale[(u + AHEAD) % S],
                             kb_begin + k + u + AHEAD, kb_begin + k + u);
      if ((!PAIRED || (u & 1)) && k + u + 1 < nkb) wait_and_barrier<YOUNGER>();
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // stray refetches must not outlive the workgroup's LDS

  store_tile<BM, SPLIT, BN>(p, acc, m0, n0, split, wave_m, wave_n, l16, q);
}

// ---- The same tile with LOADER WAVES: waves 0..7 only read LDS and multiply, LW more waves only issue the direct-to-LDS
// loads.  In the kernel above every wave's loads sit in the same in-order instruction stream as its LDS reads and MFMAs,
// and with 128-token tiles the cost of the loads ADDS to the step's own time instead of hiding under it.  Here a loader
// wave owns every LW-th group of 8 tile rows (one load instruction each) plus a copy of the tile's token-scale load, keeps
// S - 1 blocks in flight, waits until the block due next has landed (a constant vmcnt, as above) and meets the compute
// waves at the barrier that ends each K block; compute waves have nothing in vmcnt and only take the barrier.
constexpr int T_LW = 2;  // loader waves
template <int BM, int BN>
struct LoaderState {
  static constexpr int NG = (BM + BN) / 8 / T_LW;  // row groups per loader wave and K block
  static_assert((BM + BN) / 8 % T_LW == 0, "row groups divide among the loader waves");
  const uint8_t* a_base;
  const uint8_t* b_base;
  uint32_t goff[NG];  // lane's byte offset from the matrix base for row group lw + j * T_LW (rows clamped)
  const float* sa_base;
  uint32_t sa_off;
  int64_t sa_sk;
  int lw, kb_last;
};
template <int BM, int BN, bool UE8M0>
__device__ __forceinline__ void loader_issue_block(const LoaderState<BM, BN>& L, uint8_t* stage, float* scale, int kb) {
  constexpr int NG = LoaderState<BM, BN>::NG;
  kb = min(kb, L.kb_last);
#pragma unroll
  for (int j = 0; j < NG; ++j) {
    const int g = L.lw + j * T_LW;  // wave-uniform
    const uint8_t* base = (g < BM / 8 ? L.a_base : L.b_base) + (uint64_t)kb * KSTEP;
    asm volatile("" : "+s"(base));
    const uint32_t lds_addr = (uint32_t)(uintptr_t)(lptr_t)(stage + g * 8 * KSTEP);
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(L.goff[j]), "s"(base), "s"(lds_addr) : "memory");
  }
  // the tile's BM token scales: BM / 4 lanes fetch 16 bytes each (every loader wave issues it, so that all count alike)
  const float* sbase = L.sa_base + (int64_t)(UE8M0 ? kb >> 2 : kb) * L.sa_sk;
  asm volatile("" : "+s"(sbase));
  const uint32_t lds_addr = (uint32_t)(uintptr_t)(lptr_t)scale;
  uint64_t saved;
  if constexpr (BM == 128)
    asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, 0xffffffff\n\ts_mov_b32 m0, %3\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b64 exec, %0"
                 : "=&s"(saved) : "v"(L.sa_off), "s"(sbase), "s"(lds_addr) : "memory");
  else
    asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, 0xffff\n\ts_mov_b32 m0, %3\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b64 exec, %0"
                 : "=&s"(saved) : "v"(L.sa_off), "s"(sbase), "s"(lds_addr) : "memory");
}
template <int N>
__device__ __forceinline__ void loader_wait_and_barrier() {
  static_assert(N >= 1 && N <= 63, "vmcnt range");
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
}

template <int BM, bool SPLIT, int BN, bool UE8M0, int S>
__device__ __forceinline__ void dma3_tile_lw(const GemmParams& p, int m0, int n0, int split) {
  static_assert(BN == 128 || BN == 192 || BN == 256, "channel tile");
  static_assert(S >= 3 && S * ((BM + BN) * KSTEP + BM * 4) <= 160 * 1024, "the stages must fit the CU's LDS");
  constexpr int WM = BM / 2, MT = WM / 16, T_WN = BN / 4, T_NT = T_WN / 16;
  constexpr bool INTERLEAVED = Dma3State<BM, BN>::INTERLEAVED;
  constexpr int SB = Dma3State<BM, BN>::SB;
  constexpr int LPB = LoaderState<BM, BN>::NG + 1;  // loads per loader wave and K block
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kb_begin = split * p.kb_per_split;
  const int kb_end = min(p.kb_total, kb_begin + p.kb_per_split);
  const int nkb = kb_end - kb_begin;

  __shared__ __attribute__((aligned(1024))) uint8_t t_stage[S][(BM + BN) * KSTEP];
  __shared__ __attribute__((aligned(256))) float t_scale[S][BM];

  if (wave >= 8) {
    // ================= loader wave =================
    LoaderState<BM, BN> L;
    L.lw = wave - 8;
    L.kb_last = kb_end - 1;
    L.a_base = p.a, L.b_base = p.b;
    const int lrow = lane >> 3;
    const int chunk_byte = ((lane & 7) ^ lrow) * 16;  // lands swizzled by (row & 7)
#pragma unroll
    for (int j = 0; j < LoaderState<BM, BN>::NG; ++j) {
      const int row = (L.lw + j * T_LW) * 8 + lrow;
      if (row < BM) L.goff[j] = (uint32_t)((int64_t)min(m0 + row, p.M - 1) * p.lda + chunk_byte);
      else L.goff[j] = (uint32_t)((int64_t)min(n0 + row - BM, p.N - 1) * p.ldb + chunk_byte);
    }
    L.sa_base = p.sa, L.sa_sk = p.sa_sk;
    L.sa_off = (uint32_t)min(m0 + (lane & (BM / 4 - 1)) * 4, (p.M - 1) & ~3) * 4u;
#pragma unroll
    for (int b = 0; b < S - 1; ++b) loader_issue_block<BM, BN, UE8M0>(L, t_stage[b], t_scale[b], kb_begin + b);
    loader_wait_and_barrier<(S - 2) * LPB>();  // block 0 has landed
    int k = 0;
    for (; k + S - 1 < nkb; k += S) {
#pragma unroll
      for (int u = 0; u < S; ++u) {
        loader_issue_block<BM, BN, UE8M0>(L, t_stage[(u + S - 1) % S], t_scale[(u + S - 1) % S], kb_begin + k + u + S - 1);
        loader_wait_and_barrier<(S - 2) * LPB>();  // block k + u + 1 has landed
      }
    }
#pragma unroll
    for (int u = 0; u < S - 1; ++u) {
      if (k + u < nkb) {
        loader_issue_block<BM, BN, UE8M0>(L, t_stage[(u + S - 1) % S], t_scale[(u + S - 1) % S], kb_begin + k + u + S - 1);
        if (k + u + 1 < nkb) loader_wait_and_barrier<(S - 2) * LPB>();
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no refetch may outlive the workgroup's LDS
    return;
  }

  // ================= compute wave =================
  const int wave_m = wave >> 2, wave_n = wave & 3;
  const int l16 = lane & 15, q = lane >> 4;
  Dma3State<BM, BN> s;
  s.wave = wave;
  s.kb_last = kb_end - 1;
  {
    const int trow = wave_m * WM + l16, crow = BM + wave_n * (INTERLEAVED ? 16 : T_WN) + l16;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      s.tok_off[h] = trow * KSTEP + (((q + 4 * h) ^ (trow & 7)) << 4);
      s.ch_off[h] = crow * KSTEP + (((q + 4 * h) ^ (crow & 7)) << 4);
    }
    s.sc_off = (wave_m * WM + l16) * 4;
  }
#pragma unroll
  for (int b = 0; b < SB; ++b) {
    const int first = INTERLEAVED ? n0 + 64 * b : n0 + wave_n * T_WN;
    s.sb_ptr[b] = (cfloat_ptr)(p.sb + (int64_t)__builtin_amdgcn_readfirstlane(UE8M0 ? min(first, p.N - 1) : min(first, p.N - 1) / 128) * p.sb_sn);
  }
  s.sb_sk = p.sb_sk;

  float acc[T_NT][MT][4];
#pragma unroll
  for (int i = 0; i < T_NT; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.f;

  auto sb_of = [&](int kb, float (&v)[SB]) {
#pragma unroll
    for (int b = 0; b < SB; ++b) v[b] = s.sb_ptr[b][(int64_t)(UE8M0 ? kb >> 2 : kb) * s.sb_sk];
  };
  asm volatile("s_barrier" ::: "memory");  // block 0 has landed (the loaders waited for it)
  int k = 0;
  for (; k + S - 1 < nkb; k += S) {
    float sbv[S][SB];
#pragma unroll
    for (int u = 0; u < S; ++u) sb_of(kb_begin + k + u, sbv[u]);
#pragma unroll
    for (int u = 0; u < S; ++u) {
      k_block<BM, BN, UE8M0, 0>(s, t_stage[u], t_scale[u], sbv[u], acc, nullptr, nullptr, 0, kb_begin + k + u);
      asm volatile("s_barrier" ::: "memory");
    }
  }
#pragma unroll
  for (int u = 0; u < S - 1; ++u) {
    if (k + u < nkb) {
      float sbl[SB];
      sb_of(kb_begin + k + u, sbl);
      k_block<BM, BN, UE8M0, 0>(s, t_stage[u], t_scale[u], sbl, acc, nullptr, nullptr, 0, kb_begin + k + u);
      if (k + u + 1 < nkb) asm volatile("s_barrier" ::: "memory");
    }
  }

  store_tile<BM, SPLIT, BN>(p, acc, m0, n0, split, wave_m, wave_n, l16, q);
}

template <int BM, bool SPLIT, int BN, bool UE8M0, int S>
__global__ __launch_bounds__(T_THREADS + 64 * T_LW) void fp8_gemm_dma3_lw_kernel(const GemmParams p) {
  const TileCoord tc = tile_of_block(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n);
  dma3_tile_lw<BM, SPLIT, BN, UE8M0, S>(p, tc.tile_m * BM, tc.tile_n * BN, tc.split);
}

// ---- The 64-token tile for the one-call linear at decode sizes (M <= 16, K unsplit): the tokens arrive unquantized
// (p.x16, bf16 or fp16) and four more waves, the PRODUCERS, quantize the 16 x 128 values of a K block into the stage's token rows
// and scale slots - the arithmetic of the group quantizer's reference path (quantize_group_lane), so the result equals
// quantizer launch + GEMM bit for bit - while waves 0..7 load the weight rows and multiply as above.  A producer requests
// the raw tokens four blocks ahead of the one it quantizes (one 16-byte load per lane and block, its own vmcnt), writes S - 1 blocks ahead of
// the one being multiplied, and meets the others at every block's barrier.  Token rows 16..63 of a stage are never written:
// what they hold only reaches accumulators of rows that are not stored.
constexpr int T_PW = 4;  // producer waves of the fused quantizer
template <int BN, int S>
__device__ __forceinline__ void dma3_tile_q(const GemmParams& p, int n0) {
  constexpr int BM = 64;
  static_assert(S >= 3 && S * ((BM + BN) * KSTEP + BM * 4) <= 160 * 1024, "the stages must fit the CU's LDS");
  constexpr int LOADS = Dma3State<BM, BN>::LOADS, LOADS_W = LOADS - BM / 64;  // weight-row loads per wave and block
  constexpr bool INTERLEAVED = Dma3State<BM, BN>::INTERLEAVED;
  constexpr int SB = Dma3State<BM, BN>::SB, WM = BM / 2, MT = WM / 16, T_WN = BN / 4, T_NT = T_WN / 16;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nkb = p.kb_total, kb_last = p.kb_total - 1;

  __shared__ __attribute__((aligned(1024))) uint8_t t_stage[S][(BM + BN) * KSTEP];
  __shared__ __attribute__((aligned(256))) float t_scale[S][BM];

  if (wave >= 8) {
    // ================= producer wave pw: tokens 4 pw .. 4 pw + 3 =================
    // (one wave quantizing all sixteen tokens of a block takes ~1.3 us of dependent arithmetic per block, more than the block's
    // multiplication: 78 against 50 us on K=7168 -> N=36864; four waves take a quarter each)
    const int pw = wave - 8;
    const int gl = lane & 15, r4 = lane >> 4;  // 16 lanes per (token, block) group; four tokens per wave
    const int m = pw * 4 + r4;                 // the stage row this lane's group goes to; rows past M repeat the last token
    const bool active = pw * 4 < p.M;          // a wave whose tokens all lie past M only keeps the barriers
    const uint16_t* xrow = reinterpret_cast<const uint16_t*>(p.x16) + (int64_t)min(m, p.M - 1) * p.ldx + gl * 8;
    auto request = [&](int kb, u32x4& raw) {
      const uint16_t* src = xrow + (int64_t)min(kb, kb_last) * KSTEP;
      asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(raw) : "v"(src) : "memory");
    };
    auto produce = [&](int stage, const u32x4& raw) {
      float sc;
      const u32x2 codes = quantize_group_lane(raw, p.x_dtype, p.x_by_reciprocal != 0, sc);
      *reinterpret_cast<u32x2*>(&t_stage[stage][m * KSTEP + (((gl >> 1) ^ (m & 7)) << 4) + (gl & 1) * 8]) = codes;
      if (gl == 0) t_scale[stage][m] = sc;
    };
    // A ring of R registers keeps the raw tokens of the next R blocks in flight: one is quantized into its stage, then
    // requested again for the block R further on (a register that a load is still writing cannot be copied, so the loop is
    // unrolled over the ring).  Step b produces block b into stage b % S; from step S - 2 on (blocks 0 .. S-2 are in LDS) every
    // step ends at a barrier: the first is the one the other waves pass before block 0, the j-th after it ends their block j - 1,
    // so block b is written after the barrier that ends block b - S, the last reader of its stage.
    constexpr int R = 4;
    static_assert(R == 4, "the wait below is written for a ring of four loads");
    u32x4 ring[R];
    if (active) {
#pragma unroll
      for (int u = 0; u < R; ++u) request(u, ring[u]);
    }
    const int steps = nkb + S - 2;
    int st = 0;
    for (int b = 0; b < steps; b += R) {
#pragma unroll
      for (int u = 0; u < R; ++u) {
        if (b + u < steps) {
          if (active) {
            asm volatile("s_waitcnt vmcnt(3)" : "+v"(ring[u])::"memory");  // the oldest of the R loads in flight
            produce(st, ring[u]);
            st = st + 1 == S ? 0 : st + 1;
            request(b + u + R, ring[u]);
          }
          if (b + u >= S - 2) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        }
      }
    }
    if (nkb % S == 0) asm volatile("s_barrier" ::: "memory");  // the other waves' barrier after the last block of a whole trip
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    return;
  }

  // ================= waves 0..7: weight loads and arithmetic =================
  const int wave_m = wave >> 2, wave_n = wave & 3;
  const int l16 = lane & 15, q = lane >> 4;
  Dma3State<BM, BN> s;
  s.wave = wave;
  s.kb_last = kb_last;
  s.a_base = p.b;  // (token rows are not loaded; a valid address all the same)
  s.b_base = p.b;
  {
    const int lrow = lane >> 3;
    const int chunk_byte = ((lane & 7) ^ lrow) * 16;
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int row = i * 64 + wave * 8 + lrow;
      s.goff[i] = row < BM ? 0u : (uint32_t)((int64_t)min(n0 + row - BM, p.N - 1) * p.ldb + chunk_byte);
    }
    const int trow = wave_m * WM + l16, crow = BM + wave_n * (INTERLEAVED ? 16 : T_WN) + l16;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      s.tok_off[h] = trow * KSTEP + (((q + 4 * h) ^ (trow & 7)) << 4);
      s.ch_off[h] = crow * KSTEP + (((q + 4 * h) ^ (crow & 7)) << 4);
    }
    s.sc_off = (wave_m * WM + l16) * 4;
  }
  s.sa_base = p.sb, s.sa_off = 0, s.sa_sk = 0;  // (token scales are not loaded)
#pragma unroll
  for (int b = 0; b < SB; ++b) {
    const int first = INTERLEAVED ? n0 + 64 * b : n0 + wave_n * T_WN;
    s.sb_ptr[b] = (cfloat_ptr)(p.sb + (int64_t)__builtin_amdgcn_readfirstlane(min(first, p.N - 1) / 128) * p.sb_sn);
  }
  s.sb_sk = p.sb_sk;
  constexpr int YOUNGER = (S - 2) * LOADS_W;

  float acc[T_NT][MT][4];
#pragma unroll
  for (int i = 0; i < T_NT; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.f;

#pragma unroll
  for (int b = 0; b < S - 1; ++b)
#pragma unroll
    for (int i = BM / 64; i < LOADS; ++i) issue_one<BM, BN, false>(s, i, t_stage[b], t_scale[b], b);
  wait_and_barrier<YOUNGER>();  // the weight rows of block 0 have landed; the producer has written blocks 0 .. S-2

  auto sb_of = [&](int kb, float (&v)[SB]) {
#pragma unroll
    for (int b = 0; b < SB; ++b) v[b] = s.sb_ptr[b][(int64_t)kb * s.sb_sk];
  };
  int k = 0;
  for (; k + S - 1 < nkb; k += S) {
    float sbv[S][SB];
#pragma unroll
    for (int u = 0; u < S; ++u) sb_of(k + u, sbv[u]);
#pragma unroll
    for (int u = 0; u < S; ++u) {
      k_block<BM, BN, false, 2>(s, t_stage[u], t_scale[u], sbv[u], acc, t_stage[(u + S - 1) % S], t_scale[(u + S - 1) % S], k + u + S - 1, k + u);
      wait_and_barrier<YOUNGER>();  // unconditional (a condition here makes the compiler sink arithmetic across blocks): when K
                                    // is a whole number of trips this is one barrier past the last block, which the producers match
    }
  }
#pragma unroll
  for (int u = 0; u < S - 1; ++u) {
    if (k + u < nkb) {
      float sbl[SB];
      sb_of(k + u, sbl);
      k_block<BM, BN, false, 2>(s, t_stage[u], t_scale[u], sbl, acc, t_stage[(u + S - 1) % S], t_scale[(u + S - 1) % S], k + u + S - 1, k + u);
      if (k + u + 1 < nkb) wait_and_barrier<YOUNGER>();
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // stray refetches must not outlive the workgroup's LDS
  store_tile<BM, false, BN>(p, acc, 0, n0, 0, wave_m, wave_n, l16, q);
}

template <int BN, int S>
__global__ __launch_bounds__(T_THREADS + 64 * T_PW) void fp8_gemm_dma3_q_kernel(const GemmParams p) {
  const TileCoord tc = tile_of_block(blockIdx.x, gridDim.x, 1, p.tiles_n);
  dma3_tile_q<BN, S>(p, tc.tile_n * BN);
}

template <int BM, bool SPLIT, int BN, bool UE8M0 = false, int S = 3>
__global__ __launch_bounds__(T_THREADS) void fp8_gemm_dma3_kernel(const GemmParams p) {
  const TileCoord tc = tile_of_block(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n);
  dma3_tile<BM, SPLIT, BN, UE8M0, S>(p, tc.tile_m * BM, tc.tile_n * BN, tc.split);
}

// Grouped problems (see GroupedParams): the workgroup's token tile comes from the table the plan kernel wrote, the
// operand bases move to that tile's expert, and the ordinary tile runs.
template <int BM>
__global__ __launch_bounds__(T_THREADS) void fp8_grouped_dma3_kernel(const GroupedParams gp) {
  GemmParams p;
  int m0, tile_n;
  if (!grouped_tile_of_block(gp, p, m0, tile_n)) return;  // the whole workgroup leaves before any barrier
  dma3_tile<BM, false>(p, m0, tile_n * T_BN, 0);
}

// Stages per tile shape.  A 64 x 128 tile's three stages take 73.5 KB, so two such workgroups share a CU and keep four blocks
// in flight between them; where a launch has at most one workgroup per CU it runs six stages instead (one barrier per two
// blocks).  64 x 192 and 128 x 128 tiles (32 KB a stage) have the CU to themselves either way: four stages.  Measured, us,
// three stages / more: K=7168 -> N=576 at M=2048 29.0 / 26.3, K=4096 -> N=14336 at M=48 24.5 / 23.1, K=7168 -> N=4096 at
// M=512 25.8 / 24.3, K=18432 -> N=7168 at M=32 33.7 / 32.8, at M=64 37.9 / 37.3; no change (within 0.3 us) for ten other
// shapes: these tiles are bound by the step's own chain of LDS reads, MFMAs and the barrier more than by load latency.
constexpr int stages_of(int bm, int bn, bool own_cu) { return bm + bn == 192 ? (own_cu ? 6 : 3) : bm + bn == 256 ? 4 : 3; }

template <int BM, int BN, bool UE8M0 = false>
int launch_bm(GemmParams& p, hipStream_t stream, const char* what) {
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n * p.splits));
  if constexpr (BM == 128) {
    // 128-token tiles: compute waves + loader waves (1-5 % over every wave loading for itself, on all sixteen shapes
    // measured: K=7168 -> N=36864 at M=128 65.5 -> 62.6 us, K=7168 -> N=4096 at M=1024 39.1 -> 37.2, K=7168 -> N=16384 at
    // M=300 59.8 -> 57.4, K=18432 -> N=7168 at M=300 75.5 -> 72.8)
    constexpr int S = stages_of(BM, BN, true);
    if (p.splits > 1) hipLaunchKernelGGL((fp8_gemm_dma3_lw_kernel<BM, true, BN, UE8M0, S>), grid, dim3(T_THREADS + 64 * T_LW), 0, stream, p);
    else hipLaunchKernelGGL((fp8_gemm_dma3_lw_kernel<BM, false, BN, UE8M0, S>), grid, dim3(T_THREADS + 64 * T_LW), 0, stream, p);
  } else if (BM + BN == 192 && (int64_t)p.tiles_m * p.tiles_n * p.splits > NUM_CUS) {
    constexpr int S = stages_of(BM, BN, false);
    if (p.splits > 1) hipLaunchKernelGGL((fp8_gemm_dma3_kernel<BM, true, BN, UE8M0, S>), grid, dim3(T_THREADS), 0, stream, p);
    else hipLaunchKernelGGL((fp8_gemm_dma3_kernel<BM, false, BN, UE8M0, S>), grid, dim3(T_THREADS), 0, stream, p);
  } else {
    constexpr int S = stages_of(BM, BN, true);
    if (p.splits > 1) hipLaunchKernelGGL((fp8_gemm_dma3_kernel<BM, true, BN, UE8M0, S>), grid, dim3(T_THREADS), 0, stream, p);
    else hipLaunchKernelGGL((fp8_gemm_dma3_kernel<BM, false, BN, UE8M0, S>), grid, dim3(T_THREADS), 0, stream, p);
  }
  return check_launch(what);
}

}  // namespace

// Tile shape (64 or 128 tokens x 256 or 128 channels) and split count for this kernel.  One workgroup per CU fits (the
// LDS stages are sized for the widest tile).  Narrow channel tiles do half the multiplications of a block in 0.6 of the
// time, but they double the workgroups without a K split, i.e. without fp32 partial sums: they win for few channels and
// long K (K=18432 -> N=7168 at M=128: 52.7 -> 46.7 us; K=7168 -> N=4096 at M=512: 34.4 -> 24.5 us; N=576 at M=4096:
// 35.7 -> 31.0 us) and lose where 256-channel tiles already give a round's worth of workgroups.
//
// The choice minimises a time model fitted to measurements on this part (24 shapes, M = 32 .. 4096, every tile height
// and split count; it names the measured best or a choice within 5 % of it for 22 of them, within 12 % for the others):
//   * a workgroup spends per K block the largest of
//       - the tile's own time when operands come from L2: 0.88 us for 128 token rows, 0.58 us for 64 (0.52 / 0.40 with
//         128 channels, 0.68 / 0.50 with 192; x 1.2 in a round that keeps more than 200 CUs busy; the INT8 kernel: 1.14 / 0.71 / 0.64 / 0.44);
//       - a latency floor when the weight comes from HBM (two blocks in flight per CU): 1.2 us / 1.0 us (1.0 / 0.75 with 192 channels, 0.7 / 0.51 with
//         128 channels; INT8: 0.96 / 0.68 / 0.59 / 0.54), times 1.2 for weight rows longer than 8 KB;
//       - its share of the HBM stream: (concurrent workgroups) x (HBM bytes per workgroup and block) / 5.5 TB/s, where
//         weight rows are shared in L2 by up to 8 token tiles and token rows by up to 8 channel tiles;
//   * a workgroup runs kb_per + 2 blocks (pipeline fill), and rounds of up to 256 workgroups follow each other;
//   * a split adds the fp32 partial tiles written and read back (8 * splits * M * N bytes at 5.5 TB/s) and
//     8 + 0.25 * splits us for the second launch and its tail.
// So 144 workgroups streaming a weight unsplit beat 432 that split K in three (measured at M = 32 and 64 on K = 7168 ->
// N = 36864: 58 against 65 us): with all CUs busy the HBM stream, not the number of workgroups, is the limit, and the
// partial sums only add traffic.
//
// `efficiency` is the best value over all choices of an older byte-model score, kept because the dispatcher's threshold
// for preferring another kernel at M < 256 was set with it:
//   balance * useful_bytes / (useful_bytes + partial_bytes) * kb_per / (kb_per + 2) * (0.65 for 64-row tiles at M > 128)
namespace {
double dma3_model_us(int64_t M, int64_t N, int64_t kb_total, int bm, int bn, int sp, bool is_int8) {
  const RouteConstants& rc = route_constants();
  const double HBM_BYTES_PER_US = rc.dma3_hbm_bytes_per_us;
  const int64_t per = (kb_total + sp - 1) / sp;
  const int64_t tm = (M + bm - 1) / bm, tn = (N + bn - 1) / bn;
  // the tile's own time per K block and the latency floor, in the order 128x256, 64x256, 128x128, 64x128, 128x192, 64x192
  // (the INT8 kernel of the same structure has its own); the numbers and where they come from: route_constants.h
  const int shape = (bn == 256 ? 0 : bn == 128 ? 2 : 4) + (bm == 128 ? 0 : 1);  // ..., 128x192, 64x192 (FP8 only)
  const double t_tile = rc.dma3_tile_us[is_int8][shape];
  const double hbm_per_block = (double)(bn * KSTEP) / (double)std::min<int64_t>(tm, 8) + (double)(bm * KSTEP) / (double)std::min<int64_t>(tn, 8);
  // latency floor while the weight streams from HBM: with 256 or 192 channels per tile when at most two token tiles share
  // it, with 128 when nobody does (rows more than 8 KB apart cost more)
  const bool streams = hbm_per_block >= (bn == 192 ? 12288.0 : 16384.0);
  const double t_latency = streams ? rc.dma3_latency_us[is_int8][shape] * (kb_total > 64 ? rc.dma3_long_row_factor : 1.0) : 0.0;
  double t = 0.0;
  for (int64_t left = tm * tn * sp; left > 0;) {
    const int64_t c = std::min<int64_t>(left, 256);
    left -= c;
    // with (nearly) every CU multiplying, the clock drops
    const double t_own = t_tile * (c > 200 ? rc.dma3_busy_chip_factor : 1.0);
    t += (double)(per + 2) * std::max(std::max(t_own, t_latency), (double)c * hbm_per_block / HBM_BYTES_PER_US);
  }
  if (sp > 1) t += 8.0 * sp * (double)M * (double)N / HBM_BYTES_PER_US + rc.dma3_split_fixed_us + rc.dma3_split_per_split_us * sp;
  return t;
}
}  // namespace

int dma3_stages(int bm, int bn, int64_t workgroups) { return stages_of(bm, bn, workgroups <= NUM_CUS); }

Dma3Plan dma3_plan(int64_t M, int64_t N, int64_t K, bool is_int8) {
  Dma3Plan pl;
  const int64_t kb_total = (K + KSTEP - 1) / KSTEP;
  const double useful = (double)N * K + (double)M * K + 2.0 * M * N;
  const int max_split = (N % 4 == 0) ? 16 : 1;  // the reduce kernel works on aligned quads of one row
  double best_time = 1e30;
  pl.bm = 128, pl.bn = T_BN, pl.splits = 1, pl.efficiency = 0.0;
  for (int bn = T_BN; bn >= 128; bn -= 64) {
    if (bn == 192 && is_int8) continue;  // the INT8 kernel's 32-channel MFMA tiles do not divide 192 / 4
    for (int bm = 64; bm <= 128; bm += 64) {
      if (M <= 64 && bm == 128) break;                 // a second half tile of padding rows buys nothing
      const double tile_factor = (bm == 64 && M > 128) ? route_constants().dma3_small_tile_factor : 1.0;
      const int64_t tiles = ((M + bm - 1) / bm) * ((N + T_BN - 1) / T_BN);
      for (int sp = 1; sp <= max_split; ++sp) {
        const int64_t per = (kb_total + sp - 1) / sp;
        if (sp > 1 && per < 4) break;
        if ((kb_total + per - 1) / per != sp) continue;  // some split would get no work
        const double t = dma3_model_us(M, N, kb_total, bm, bn, sp, is_int8);
        if (t < best_time) best_time = t, pl.splits = sp, pl.bm = bm, pl.bn = bn;
        if (bn != T_BN) continue;  // the byte-model score below is defined on 256-channel tiles
        const int64_t wgs = tiles * sp;
        const int64_t rounds = (wgs + 255) / 256;
        const double balance = (double)wgs / (double)(rounds * 256);
        const double partial = sp > 1 ? 8.0 * sp * M * N : 0.0;
        pl.efficiency = std::max(pl.efficiency, balance * useful / (useful + partial) * (double)per / (double)(per + 2) * tile_factor);
      }
    }
  }
  pl.kb_per_split = (int)((kb_total + pl.splits - 1) / pl.splits);
  pl.time_us = best_time;
  return pl;
}

int launch_fp8_grouped_dma3(GroupedParams& gp, int bm, hipStream_t stream, const char* what) {
  gp.g.tiles_n = (gp.g.N + T_BN - 1) / T_BN;
  gp.g.splits = 1, gp.g.kb_per_split = gp.g.kb_total;
  const dim3 grid((unsigned)(gp.max_tiles_m * gp.g.tiles_n));
  if (bm == 64)
    hipLaunchKernelGGL(fp8_grouped_dma3_kernel<64>, grid, dim3(T_THREADS), 0, stream, gp);
  else
    hipLaunchKernelGGL(fp8_grouped_dma3_kernel<128>, grid, dim3(T_THREADS), 0, stream, gp);
  return check_launch(what);
}

int launch_fp8_dma3(GemmParams& p, int bm, int bn, hipStream_t stream, const char* what) {
  if (bn == 128) return bm == 64 ? launch_bm<64, 128>(p, stream, what) : launch_bm<128, 128>(p, stream, what);
  if (bn == 192) return bm == 64 ? launch_bm<64, 192>(p, stream, what) : launch_bm<128, 192>(p, stream, what);
  return bm == 64 ? launch_bm<64, 256>(p, stream, what) : launch_bm<128, 256>(p, stream, what);
}

// One-call linear at decode sizes: p.x16 / p.ldx / p.x_dtype describe the unquantized tokens (M <= 16, 16-byte aligned rows),
// K unsplit, one 64-token tile per workgroup; p.a and p.sa are not read.
int launch_fp8_dma3_quant(GemmParams& p, int bn, hipStream_t stream, const char* what) {
  if (p.M > 16 || p.x16 == nullptr || p.splits != 1) {
    set_error("%s: the fused quantizer of the mid-M kernel takes up to 16 unquantized tokens and an unsplit K", what);
    return MI355_ERR_UNSUPPORTED;
  }
  p.tiles_m = 1;
  p.tiles_n = (p.N + bn - 1) / bn;
  const dim3 grid((unsigned)p.tiles_n), block(T_THREADS + 64 * T_PW);
  if (bn == 128) hipLaunchKernelGGL((fp8_gemm_dma3_q_kernel<128, 6>), grid, block, 0, stream, p);
  else if (bn == 192) hipLaunchKernelGGL((fp8_gemm_dma3_q_kernel<192, 4>), grid, block, 0, stream, p);
  else hipLaunchKernelGGL((fp8_gemm_dma3_q_kernel<256, 3>), grid, block, 0, stream, p);
  return check_launch(what);
}

// The same kernels for packed power-of-two (UE8M0) scales on both operands, applied by the MFMA (see dma3_tile).
int launch_fp8_dma3_ue8m0(GemmParams& p, int bm, int bn, hipStream_t stream, const char* what) {
  if (bn == 128) return bm == 64 ? launch_bm<64, 128, true>(p, stream, what) : launch_bm<128, 128, true>(p, stream, what);
  if (bn == 192) return bm == 64 ? launch_bm<64, 192, true>(p, stream, what) : launch_bm<128, 192, true>(p, stream, what);
  return bm == 64 ? launch_bm<64, 256, true>(p, stream, what) : launch_bm<128, 256, true>(p, stream, what);
}

}  // namespace mi355
