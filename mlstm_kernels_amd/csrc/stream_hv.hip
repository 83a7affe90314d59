// Streaming form of the chunk-parallel kernels whose output tile spans value columns (forward output H, gradient dV):
// the same arithmetic as par_hv.hip (see there for the formulas and the state-stride algebra), organised around the
// two resources that bind it on this chip: HBM bandwidth and the LDS read port of a CU (about 128 bytes per clock;
// every matrix instruction fed from LDS costs 1 KB of it at a 2 x 2 register blocking).
//
//   * One PERSISTENT workgroup per CU (twelve waves) walks its share of the work items; an item is one chunk of 128
//     positions x 512 value columns of one (batch, head), so the gated score blocks of a chunk are computed once.
//   * The waves have two roles.  Four PRODUCER waves do nothing but move data: every operand of every item -- the 128
//     resident rows (Q forward, K for dV), the kept state as ready-made operand fragments, the rows of the source
//     chunks for the scores and for the output product -- is cut into slabs of 32 KB, and the producers always have two
//     slabs (64 KB per CU) on their way from memory in registers, across item boundaries, so the memory pipe does not
//     drain while an item starts up or is written out.  Eight CONSUMER waves own 64 positions x 128 columns each (128
//     accumulator registers: three waves per SIMD leave 168 registers a wave), read operand fragments from LDS (six
//     fragments feed eight matrix instructions), gate the score blocks and write the output; they never wait for
//     global memory.
//   * The two roles meet at ONE barrier per slab: after barrier g the consumers work on slab g while the producers
//     write slab g+1 into the other ring slot and request slab g+3.  Both roles walk the same item list with the same
//     number of steps per item (10 + 6 per source chunk), so they pass the same number of barriers by construction.
//   * The output of an item is written while the resident rows of the next item arrive (those two steps carry no
//     operand the consumers could use), transposed through the ring slots and the score block, which are idle then.
//
// Step sequence of an item (s source chunks, the own chunk last):
//   2 x resident rows (64 rows each, written straight into their LDS tile)
//   8 x state slab: 2 contraction steps x 16 fragment blocks of 32 value columns
//   per source chunk, per half of 64 source positions: 1 slab of 64 rows x DHQK (scores, gated into the score block
//   in the same step), 2 slabs of 32 rows x 512 value columns (output product)
// Register set and ring slot alternate from step to step and every source chunk has an even number of steps, so both
// are compile-time constants everywhere.
// Supported: DHQK = 256, DHHV a multiple of 512, S a multiple of 128, no head norm; everything else runs par_hv.hip.
#include "common.h"
#include "kernels.h"

namespace mlstm {
namespace {

struct HvItem {
  int bh, c, ch;               // (batch * head), chunk, group of 512 value columns
  int slot;                    // kept boundary state the chunk uses
  int sc_first, sc_step, nsc;  // source chunks: sc_first, sc_first + sc_step, ... (nsc of them, the own chunk last)
};

// Work item of workgroup `vid` in round `round`.  Consecutive workgroups take consecutive items (neighbouring chunks
// share rows and kept states through the L2 of their XCD); the assignment rotates by one item per round so that a
// workgroup does not always get the chunks with the same number of source chunks.
template <bool IS_DV>
__device__ __forceinline__ bool hv_decode(HvItem& it, int round, int vid, int G, int n_items, int NC, int NCH, int stride) {
  const int rot = (vid + round) % G;
  const long long idx = (long long)round * G + rot;
  if (idx >= n_items) return false;
  const int i = (int)idx;
  it.ch = i % NCH;
  const int rest = i / NCH;
  it.c = rest % NC;
  it.bh = rest / NC;
  it.slot = it.c / stride;
  if (IS_DV) {
    const int hi = min(it.slot * stride + stride - 1, NC - 1);
    it.sc_first = hi;
    it.sc_step = -1;
    it.nsc = hi - it.c + 1;
  } else {
    it.sc_first = it.slot * stride;
    it.sc_step = 1;
    it.nsc = it.c - it.sc_first + 1;
  }
  return true;
}

constexpr float kLog2e = 1.4426950408889634f;

}  // namespace

// NORM (forward, DHHV = 512: a work item then holds complete rows of H): the multi-head layer / rms norm over the value
// columns is applied when the rows are rounded, as an affine map of the accumulators.
template <bool IS_DV, bool F16, bool NORM = false>
__global__ __launch_bounds__(768) void stream_hv_kernel(ParHvArgs a, int n_items, int n_rounds) {
  static_assert(!(IS_DV && NORM), "the head norm belongs to the forward");
  constexpr int DHQK = 256;
  constexpr int QS = DHQK + 8;   // resident rows [128][DHQK] and score-operand slabs [64][DHQK], fragment order
  constexpr int VS = 512 + 16;   // value-operand slab: 32 rows x 512 value columns, row-major
  constexpr int PSS = 64 + 8;    // gated score block P[n][o]: 128 positions x 64 source positions
  constexpr int SLOT = 64 * QS;  // elements per ring slot (the largest slab kind)
  constexpr int ND = DHQK / 16;
  static_assert(32 * VS <= SLOT && 16384 <= SLOT, "every slab kind fits a ring slot");
  extern __shared__ __align__(16) unsigned char smem_raw[];
  // [resident rows | ring slot 0 | score block | ring slot 1 | vectors]: the epilogue stages through everything between
  // the resident rows and the vectors in its first step and through score block + slot 1 in its second (slot 0 then
  // receives the first state slab)
  uint16_t* const Ns = (uint16_t*)smem_raw;
  uint16_t* const Ring0 = Ns + 128 * QS;
  uint16_t* const Ps = Ring0 + SLOT;
  uint16_t* const Ring1 = Ps + 128 * PSS;
  float* const rows = (float*)(Ring1 + SLOT);  // [4][128] partial row sums of the own chunk's scores (forward)
  float* const inv = rows + 4 * 128;           // [128] forward: 1 / (row normaliser + eps)
  float* const nperm = inv + 128;              // [DHQK] forward: n before the chunk, fragment order
  float* const ovec = nperm + DHQK;            // [64] gate vector of the source half: w_j (forward) / u_t (dV)
  float* const orho = ovec + 64;               // [64] dV: rho_t of the source half
  float* const denq = orho + 64;               // [128] forward: bbar_t / sqrt(d) * (q_t . n_prev), the inter-chunk part of the denominator
  float* const mcv = denq + 128;               // [128] forward: combined stabiliser of the item's positions
  float* const nst = mcv + 128;                // NORM: [4][2][128] sum and sum of squares of a row over each wave's 128 columns
  constexpr uint32_t kRing0Off = 128 * QS * 2, kRing1Off = kRing0Off + (SLOT + 128 * PSS) * 2;

  const int lane = threadIdx.x & 63;
  const int wave_all = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int G = gridDim.x;
  int vid = blockIdx.x;
  if (G % 8 == 0) vid = (vid % 8) * (G / 8) + vid / 8;  // consecutive ids share an XCD (and its L2)
  const int NC = a.NC, S = a.S, DHHV = a.DHHV, NCH = DHHV / 512, stride = a.stride;
  const size_t Sp = (size_t)NC * kChunk;
  const int NCS = (NC + stride - 1) / stride;

  if (wave_all >= 8) {
    // =========================================================================================== producer waves
    // Load step L (counted over all items of this workgroup) uses register set L % 3.  Handling it means: pass barrier
    // L - 4 (the consumers are done with slab L - 5, whose ring slot slab L - 3 goes into), write slab L - 3 from the
    // register set to LDS, request slab L into the set: three slabs are on their way at any time.  The destination in LDS travels with the data: byte offset of
    // the thread's first piece | slab kind << 20 (0 fragment-order rows, 1 state fragments, 3 value rows) | gate-vector
    // flag << 22; the thread's other seven pieces lie a fixed distance apart.
    // the loaders go first wherever a SIMD has a choice: their stores and requests after a barrier are what the next
    // step of everybody waits for (measured: 2-4 % on this kernel; in the window dQ / dK kernel it costs 2 %)
    __builtin_amdgcn_s_setprio(2);
    const int p = (wave_all - 8) * 64 + lane;  // 0 .. 255: every thread moves eight 16-byte pieces of every slab
    const char* const Xn_b = (const char*)(IS_DV ? a.K : a.Q);
    const char* const Xo_b = (const char*)(IS_DV ? a.Q : a.K);
    const char* const Xw_b = (const char*)(IS_DV ? a.dH : a.V);
    const char* const St_b = (const char*)a.states;
    const float* const ov_src = IS_DV ? a.g.u : a.g.w;
    const float* const rho_src = (IS_DV && a.use_nrow) ? a.nrow : ov_src;
    // three register sets, named by a pasted literal
    u32x4 fd0[8], fd1[8], fd2[8];
    uint32_t fw0 = 0, fw1 = 0, fw2 = 0;
    float fa0[2], fa1[2], fa2[2];
    int L = 0;
#define HV_STORE(E)                                                                                                  \
  {                                                                                                                  \
    const uint32_t w_ = fw##E;                                                                                       \
    const uint32_t kind_ = (uint32_t)__builtin_amdgcn_readfirstlane((int)((w_ >> 20) & 3));                          \
    const bool whole_ = __builtin_amdgcn_readfirstlane((int)((w_ >> 23) & 1)) == 0;                                  \
    const uint32_t d0_ = w_ & 0xFFFFFu;                                                                              \
    const uint32_t half_ = kind_ == 0 ? 16u : 8u;                                                                    \
    const uint32_t step_ = kind_ == 0 ? 8 * QS * 2 : (kind_ == 1 ? 4096 : 4 * VS * 2);                               \
    _Pragma("unroll") for (int i_ = 0; i_ < 4; ++i_) {                                                               \
      *(uint2*)(smem_raw + d0_ + i_ * step_) = make_uint2(fd##E[i_][0], fd##E[i_][1]);                               \
      *(uint2*)(smem_raw + d0_ + i_ * step_ + half_) = make_uint2(fd##E[i_][2], fd##E[i_][3]);                       \
    }                                                                                                                \
    if (whole_) {                                                                                                    \
      _Pragma("unroll") for (int i_ = 4; i_ < 8; ++i_) {                                                             \
        *(uint2*)(smem_raw + d0_ + i_ * step_) = make_uint2(fd##E[i_][0], fd##E[i_][1]);                             \
        *(uint2*)(smem_raw + d0_ + i_ * step_ + half_) = make_uint2(fd##E[i_][2], fd##E[i_][3]);                     \
      }                                                                                                              \
    }                                                                                                                \
    if (__builtin_amdgcn_readfirstlane((int)((w_ >> 22) & 1)) && p < 64) {                                           \
      ovec[p] = fa##E[0];                                                                                   \
      if (IS_DV) orho[p] = a.use_nrow ? 1.f / (fa##E[1] + a.eps) : 1.f;                                              \
    }                                                                                                                \
  }
    // base_: (batch, head) base of the operand; g0_: byte offset of the thread's first piece, gs_: distance between
    // its pieces; gi_: index of the gate-vector entry that rides along (stored only with the flag set; the other
    // slabs request an entry all the same so that every step issues the same loads); NP_: pieces per thread (8, or 4
    // for the half-size slabs of the resident rows, flagged by bit 23 of the destination word)
#define HV_PROC(E, NP_, base_, g0_, gs_, dstw_, gi_)                                                                 \
  {                                                                                                                  \
    if (L >= 4) __syncthreads();                                                                                           \
    /* piece by piece: the old content of a register goes to LDS, then the register is requested anew, so that the */ \
    /* LDS port and the vector-memory path of the CU work side by side instead of one after the other */             \
    const uint32_t w_ = fw##E;                                                                                       \
    const uint32_t kind_ = (uint32_t)__builtin_amdgcn_readfirstlane((int)((w_ >> 20) & 3));                          \
    const bool whole_ = __builtin_amdgcn_readfirstlane((int)((w_ >> 23) & 1)) == 0;                                  \
    const uint32_t d0_ = w_ & 0xFFFFFu;                                                                              \
    const uint32_t half_ = kind_ == 0 ? 16u : 8u;                                                                    \
    const uint32_t step_ = kind_ == 0 ? 8 * QS * 2 : (kind_ == 1 ? 4096 : 4 * VS * 2);                               \
    const bool st_ = L >= 3;                                                                                         \
    if (st_ && __builtin_amdgcn_readfirstlane((int)((w_ >> 22) & 1)) && p < 64) {                                    \
      ovec[p] = fa##E[0];                                                                                   \
      if (IS_DV) orho[p] = a.use_nrow ? 1.f / (fa##E[1] + a.eps) : 1.f;                                              \
    }                                                                                                                \
    fa##E[0] = ov_src[gi_];                                                                                          \
    fa##E[1] = rho_src[gi_];                                                                                         \
    _Pragma("unroll") for (int i_ = 0; i_ < 8; ++i_) {                                                               \
      if (st_ && (i_ < 4 || whole_)) {                                                                               \
        *(uint2*)(smem_raw + d0_ + i_ * step_) = make_uint2(fd##E[i_][0], fd##E[i_][1]);                             \
        *(uint2*)(smem_raw + d0_ + i_ * step_ + half_) = make_uint2(fd##E[i_][2], fd##E[i_][3]);                     \
      }                                                                                                              \
      if (i_ < (NP_)) fd##E[i_] = *(const u32x4*)((base_) + ((g0_) + i_ * (gs_)));                                             \
    }                                                                                                                \
    fw##E = (dstw_) | ((NP_) == 4 ? 1u << 23 : 0u);                                                                  \
    ++L;                                                                                                             \
  }
    HvItem it;
    for (int rd = 0; rd < n_rounds; ++rd) {
      if (!hv_decode<IS_DV>(it, rd, vid, G, n_items, NC, NCH, stride)) continue;
      // An item has 12 + 6 s steps, a multiple of three: the register set of every step is a literal.
      const uint32_t pl = (uint32_t)opaque(p);
      const uint32_t row = pl >> 5, pc = pl & 31;  // rows of 512 bytes: 32 pieces per row, 8 rows per sweep
      const size_t gown = (size_t)it.bh * Sp + (size_t)it.c * kChunk + (pl & 63);
      // fragment-order destination of piece pc inside a row (see store_perm16)
      const uint32_t permo = (pc >> 1) * 32 + 8 * (pc & 1);
      {
        // ---- resident rows, 32 per step (half-size slabs: four steps for the consumers' epilogue of the previous
        // item, and a step count per item that is a multiple of three)
        const char* const base = Xn_b + (size_t)it.bh * S * DHQK * 2;
        const uint32_t g0 = ((uint32_t)(it.c * kChunk) + row) * (DHQK * 2) + pc * 16;
        const uint32_t d0 = row * (QS * 2) + permo;
        HV_PROC(0, 4, base, g0, 8 * DHQK * 2, d0, gown)
        HV_PROC(1, 4, base, g0 + 32 * DHQK * 2, 8 * DHQK * 2, d0 + 32 * QS * 2, gown)
        HV_PROC(2, 4, base, g0 + 64 * DHQK * 2, 8 * DHQK * 2, d0 + 64 * QS * 2, gown)
        HV_PROC(0, 4, base, g0 + 96 * DHQK * 2, 8 * DHQK * 2, d0 + 96 * QS * 2, gown)
      }
      {
        // ---- state fragments: slab si holds contraction steps 2 si, 2 si + 1 of the sixteen 32-column blocks
        const char* const base = St_b + ((size_t)it.bh * NCS + it.slot) * (size_t)(DHHV / 32) * ND * 1024;
        const uint32_t f0 = pl >> 6;  // fragment of the first piece inside the slab: block f0 / 2, contraction step f0 % 2
        const uint32_t g0 = (((uint32_t)it.ch * 16 + (f0 >> 1)) * ND + (f0 & 1)) * 1024 + (pl & 63) * 16;
        const uint32_t r0 = (kRing0Off + pl * 16) | (1u << 20), r1 = (kRing1Off + pl * 16) | (1u << 20);
        HV_PROC(1, 8, base, g0, 2 * ND * 1024, r0, gown)
        HV_PROC(2, 8, base, g0 + 1 * 2048, 2 * ND * 1024, r1, gown)
        HV_PROC(0, 8, base, g0 + 2 * 2048, 2 * ND * 1024, r0, gown)
        HV_PROC(1, 8, base, g0 + 3 * 2048, 2 * ND * 1024, r1, gown)
        HV_PROC(2, 8, base, g0 + 4 * 2048, 2 * ND * 1024, r0, gown)
        HV_PROC(0, 8, base, g0 + 5 * 2048, 2 * ND * 1024, r1, gown)
        HV_PROC(1, 8, base, g0 + 6 * 2048, 2 * ND * 1024, r0, gown)
        HV_PROC(2, 8, base, g0 + 7 * 2048, 2 * ND * 1024, r1, gown)
      }
      {
        const char* const kbase = Xo_b + (size_t)it.bh * S * DHQK * 2;
        const char* const vbase = Xw_b + (size_t)it.bh * S * DHHV * 2;
        const uint32_t kd = row * (QS * 2) + permo;
        const uint32_t vrow = pl >> 6, vpc = pl & 63;  // rows of 1024 bytes: 64 pieces per row, 4 rows per sweep
        const uint32_t vd = (vrow * (VS * 2) + vpc * 16) | (3u << 20);
        for (int sci = 0; sci < it.nsc; ++sci) {
          const int sc = it.sc_first + sci * it.sc_step;
          const uint32_t t0 = (uint32_t)(sc * kChunk);
          const size_t gi = (size_t)it.bh * Sp + (size_t)sc * kChunk + (pl & 63);
          const uint32_t vg = (t0 + vrow) * (uint32_t)(DHHV * 2) + (uint32_t)it.ch * 1024 + vpc * 16;
          const uint32_t vgs = 4 * (uint32_t)DHHV * 2, vg32 = 32 * (uint32_t)DHHV * 2;
          // first half: scores -> slot 0, value rows -> slot 1 and slot 0
          HV_PROC(0, 8, kbase, (t0 + row) * (DHQK * 2) + pc * 16, 8 * DHQK * 2, (kRing0Off + kd) | (1u << 22), gi)
          HV_PROC(1, 8, vbase, vg, vgs, kRing1Off + vd, gown)
          HV_PROC(2, 8, vbase, vg + vg32, vgs, kRing0Off + vd, gown)
          // second half: the other way round
          HV_PROC(0, 8, kbase, (t0 + 64 + row) * (DHQK * 2) + pc * 16, 8 * DHQK * 2, (kRing1Off + kd) | (1u << 22), gi + 64)
          HV_PROC(1, 8, vbase, vg + 2 * vg32, vgs, kRing0Off + vd, gown)
          HV_PROC(2, 8, vbase, vg + 3 * vg32, vgs, kRing1Off + vd, gown)
        }
      }
    }
    // ---- drain: the last three slabs go to LDS, then the barriers of the consumers' last steps and of the final epilogue
    if (L > 0) {
      if (L >= 4) __syncthreads();
      HV_STORE(0)
      __syncthreads();
      HV_STORE(1)
      __syncthreads();
      HV_STORE(2)
      __syncthreads();
      __syncthreads();
      __syncthreads();
    }
#undef HV_PROC
#undef HV_STORE
  } else {
    // =========================================================================================== consumer waves
    const int wave = wave_all;
    const int tid = wave * 64 + lane;
    const int pi = wave & 1, ci = wave >> 1;  // output role: positions 64 pi .., value columns 128 ci .. of the item
    const int pb = wave & 3, kb = wave >> 2;  // score role: position block pb, source block kb of a 64-position half
    f32x16 acc[4][2], sacc;
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.f;
    HvItem it, prev;
    prev = HvItem{0, 0, 0, 0, 0, 1, 1};
    bool have_prev = false;
    // The accumulators are only ever touched in straight-line code between barriers: no matrix instruction that
    // updates them sits under a condition (dead score blocks of the own chunk are masked to zero by the gating), so
    // the compiler keeps every accumulator in one place.  The epilogue is a macro with literal block indices:
    // (normalise,) round, transpose 32 positions x (32 NMB) columns through a private staging area, coalesced
    // non-temporal stores.  STG_: staging base of this wave, MB0_: first column block, NMB_: column blocks (4 or 2).
#define HV_EPILOGUE(NB, MB0_, NMB_, STG_)                                                                            \
  {                                                                                                                  \
    const int le = opaque(lane);                                                                                     \
    const int r = le & 31, h = le >> 5;                                                                              \
    constexpr int SR = 32 * (NMB_) + 8; /* staging row */                                                            \
    uint16_t* const stg = (STG_);                                                                                    \
    float iv = IS_DV ? 1.f : inv[64 * pi + 32 * NB + r];                                                             \
    float sh = 0.f;                                                                                                  \
    if constexpr (NORM) {                                                                                            \
      /* x = acc * iv is the row of H; mean and variance over its 512 columns from the four waves' sums */            \
      const int t_ = 64 * pi + 32 * NB + r;                                                                          \
      const float t1_ = (nst[t_] + nst[256 + t_]) + (nst[512 + t_] + nst[768 + t_]);                                 \
      const float t2_ = (nst[128 + t_] + nst[384 + t_]) + (nst[640 + t_] + nst[896 + t_]);                           \
      const float ex_ = t1_ * iv * (1.f / 512.f), ex2_ = t2_ * iv * iv * (1.f / 512.f);                              \
      const float mean_ = a.head_norm == 1 ? ex_ : 0.f;                                                              \
      const float rstd_ = rsqrtf(fmaxf(ex2_ - mean_ * mean_, 0.f) + a.norm_eps);                                     \
      if (ci == 0 && h == 0) {                                                                                       \
        const size_t tg_ = (size_t)prev.bh * S + (size_t)prev.c * kChunk + t_;                                       \
        a.norm_mean[tg_] = mean_;                                                                                    \
        a.norm_rstd[tg_] = rstd_;                                                                                    \
      }                                                                                                              \
      iv *= rstd_;                                                                                                   \
      sh = -mean_ * rstd_;                                                                                           \
    }                                                                                                                \
    _Pragma("unroll") for (int mb = 0; mb < (NMB_); ++mb) _Pragma("unroll") for (int g4 = 0; g4 < 4; ++g4) {         \
      *(uint2*)(stg + r * SR + 32 * mb + 8 * g4 + 4 * h) =                                                           \
          make_uint2(pack2<F16>(__builtin_fmaf(acc[(MB0_) + mb][NB][4 * g4 + 0], iv, sh),                            \
                                __builtin_fmaf(acc[(MB0_) + mb][NB][4 * g4 + 1], iv, sh)),                           \
                     pack2<F16>(__builtin_fmaf(acc[(MB0_) + mb][NB][4 * g4 + 2], iv, sh),                            \
                                __builtin_fmaf(acc[(MB0_) + mb][NB][4 * g4 + 3], iv, sh)));                          \
    }                                                                                                                \
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");                                                           \
    __builtin_amdgcn_wave_barrier();                                                                                 \
    uint16_t* const Og = a.Out + ((size_t)prev.bh * S + (size_t)prev.c * kChunk + 64 * pi + 32 * NB) * DHHV +        \
                         prev.ch * 512 + 128 * ci + 32 * (MB0_);                                                     \
    constexpr int VPR = 4 * (NMB_); /* 16-byte vectors per row */                                                    \
    _Pragma("unroll") for (int k = 0; k < 32 * VPR / 64; ++k) {                                                      \
      const int row = le / VPR + (64 / VPR) * k, pc = le % VPR;                                                      \
      __builtin_nontemporal_store(*(const u32x4*)(stg + row * SR + pc * 8), (u32x4*)(Og + (size_t)row * DHHV + pc * 8)); \
    }                                                                                                                \
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");                                                           \
    __builtin_amdgcn_wave_barrier();                                                                                 \
  }
    for (int rd = 0; rd < n_rounds; ++rd) {
      if (!hv_decode<IS_DV>(it, rd, vid, G, n_items, NC, NCH, stride)) continue;
      const int bh = it.bh, c = it.c;
      const size_t hofs = (size_t)bh * Sp, gofs = hofs + (size_t)c * kChunk;
      const float* graw = a.g.graw + (size_t)bh * NC;
      const float* mst = a.g.mstates + (size_t)bh * (NC + 1);
      // ---- two steps while the resident rows arrive: the previous item's output leaves (the first 32 of a wave's 64
      // positions, then the other 32 in two rounds of 64 columns: the second step has less LDS to stage through), the
      // per-item vectors are requested
      float csr[2], nv, cs0r = 0.f, mcr = 0.f, np0 = 0.f, np1 = 0.f, np2 = 0.f;
      __syncthreads();
      if (have_prev) HV_EPILOGUE(0, 0, 4, Ring0 + wave * (32 * 136))
      {
        const int r = opaque(lane) & 31;
        float gsum = 0.f, xs = 1.f;
        if (IS_DV) {
          const int hi = it.sc_first;
          for (int x = c + 1; x <= hi; ++x) gsum += graw[x];
          if (hi > c) xs = __expf(gsum + mst[c + 1] - mst[hi + 1]);
        } else {
          const int lo = it.sc_first;
          for (int x = lo; x < c; ++x) gsum += graw[x];
          if (lo < c) xs = __expf(gsum + mst[lo] - mst[c]);
        }
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
          const size_t gi = gofs + 64 * pi + 32 * nb + r;
          csr[nb] = (IS_DV ? a.g.abar[gi] : a.g.bbar[gi] * a.qk_scale) * xs;
        }
        nv = (IS_DV ? a.g.w : a.g.u)[gofs + 32 * pb + r];
        if (!IS_DV) {
          const int t = opaque(tid) >> 2;
          cs0r = a.g.bbar[gofs + t] * a.qk_scale;
          mcr = a.g.mcomb[gofs + t];
          if (tid < DHQK) {
            // the scan hands n over as three partial vectors per chunk (their sum carries the full fp32 precision)
            const float* np3 = a.nstates + ((size_t)bh * NC + c) * 3 * DHQK + tid;
            np0 = np3[0];
            np1 = np3[DHQK];
            np2 = np3[2 * DHQK];
          }
        }
      }
      __syncthreads();
      if (have_prev) HV_EPILOGUE(1, 0, 4, Ring0 + wave * (32 * 136))
      __syncthreads();
      if (!IS_DV && tid < DHQK) nperm[perm16(tid)] = (np0 + np1) + np2;
      __syncthreads();
      // ---- inter-chunk product: Out^T = State^T Xn^T, two contraction steps per slab
#pragma unroll
      for (int si = 0; si < 8; ++si) {
        __syncthreads();
        if (!IS_DV) {
          if (si == 0) {
            // forward: q_t . n_prev for the denominators (four threads per position), while the resident rows are
            // all there -- the next item's rows start to arrive during this item's last step
            const int td = opaque(tid);
            const int t = td >> 2, part = td & 3;
            const uint16_t* qrow = Ns + t * QS + part * (DHQK / 4);
            const float* np = nperm + part * (DHQK / 4);
            float dot = 0.f;
#pragma unroll 1
            for (int d = 0; d < DHQK / 4; d += 8) {
              const uint4 qv = *(const uint4*)(qrow + d);
              const float4 na = *(const float4*)(np + d), nb4 = *(const float4*)(np + d + 4);
              dot += lo2<F16>(qv.x) * na.x + hi2<F16>(qv.x) * na.y + lo2<F16>(qv.y) * na.z + hi2<F16>(qv.y) * na.w;
              dot += lo2<F16>(qv.z) * nb4.x + hi2<F16>(qv.z) * nb4.y + lo2<F16>(qv.w) * nb4.z + hi2<F16>(qv.w) * nb4.w;
            }
            dot += __shfl_xor(dot, 1);
            dot += __shfl_xor(dot, 2);
            // parked in LDS until the row sums of the own chunk are complete: registers are what this kernel is short of
            if (part == 0) {
              denq[t] = cs0r * dot;
              mcv[t] = mcr;
            }
          }
        }
        if (si == 0) {
          // (after the dot product above, which runs while no accumulator is live)
#pragma unroll
          for (int mb = 0; mb < 4; ++mb)
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
              for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.f;
        }
        const int le = opaque(lane);
        const int r = le & 31, h = le >> 5;
        const uint16_t* const slab = (si & 1) ? Ring1 : Ring0;
#pragma unroll
        for (int dsl = 0; dsl < 2; ++dsl) {
          Frag A[4], B[2];
#pragma unroll
          for (int mb = 0; mb < 4; ++mb) A[mb].u = *(const uint4*)(slab + ((4 * ci + mb) * 2 + dsl) * 512 + le * 8);
#pragma unroll
          for (int nb = 0; nb < 2; ++nb)
            B[nb].u = *(const uint4*)(Ns + (64 * pi + 32 * nb + r) * QS + 16 * (2 * si + dsl) + 8 * h);
#pragma unroll
          for (int mb = 0; mb < 4; ++mb)
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) mfma32<F16>(acc[mb][nb], A[mb], B[nb]);
        }
      }
      // (kept apart from the matrix instructions around it: interleaved with them the products land in fresh
      // registers, a second copy of an accumulator tile the register file has no room for)
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) acc[mb][nb] *= csr[nb];
      __builtin_amdgcn_sched_barrier(0);

      // ---- source chunks (the own chunk last), 64 source positions at a time
      for (int sci = 0; sci < it.nsc; ++sci) {
        const int sc = it.sc_first + sci * it.sc_step;
        const bool own = sc == c;
        float gs = 0.f;  // decay between the source chunk and this chunk
        for (int x = (IS_DV ? c : sc); x < (IS_DV ? sc : c); ++x) gs += graw[x];
        // gate exponent of this lane's position; the 1/sqrt(d) of the scores rides in the exponent (lq)
        const float un = nv + (IS_DV ? -gs : gs);
        const float lq = __log2f(a.qk_scale);
#pragma unroll
        for (int kh = 0; kh < 2; ++kh) {
          // the two halves use the ring slots the other way round (three slabs per half)
          const uint16_t* const kslab = kh == 0 ? Ring0 : Ring1;
          // scores of position block pb against source block kb of this half
#pragma unroll
          for (int i = 0; i < 16; ++i) sacc[i] = 0.f;
          __syncthreads();
          {
            const int le = opaque(lane);
            const int r = le & 31, h = le >> 5;
            // blocks of the own chunk that the causal mask empties are not multiplied (their rows stay zero)
            const bool live = !own || (IS_DV ? (2 * kh + kb >= pb) : (2 * kh + kb <= pb));
            if (live) {
#pragma unroll
              for (int ds = 0; ds < ND; ++ds) {
                Frag A, B;
                A.u = *(const uint4*)(kslab + (32 * kb + r) * QS + 16 * ds + 8 * h);
                B.u = *(const uint4*)(Ns + (32 * pb + r) * QS + 16 * ds + 8 * h);
                mfma32<F16>(sacc, A, B);
              }
            }
            // gate, mask, round and write P as Ps[n][o]; forward: fp32 row sums over the own chunk's positions
            const int n = 32 * pb + r;  // position inside the chunk
            float rsum = 0.f;
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
              const int ol = 32 * kb + 8 * g4 + 4 * h;  // source position inside the half
              const float4 xo = *(const float4*)(ovec + ol);
              const float xov[4] = {xo.x, xo.y, xo.z, xo.w};
              float rho[4] = {1.f, 1.f, 1.f, 1.f};
              if (IS_DV) {
                const float4 rr = *(const float4*)(orho + ol);
                rho[0] = rr.x; rho[1] = rr.y; rho[2] = rr.z; rho[3] = rr.w;
              }
              float pv[4];
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                const int o = 64 * kh + ol + q;
                // exp(u_t - w_j + G) / sqrt(d) as one power of two
                const float e2 = __builtin_amdgcn_exp2f(__builtin_fmaf(IS_DV ? (xov[q] - un) : (un - xov[q]), kLog2e, lq));
                const bool keep = !own || (IS_DV ? (n <= o) : (o <= n));
                float val = sacc[4 * g4 + q] * e2;
                if (IS_DV) val *= rho[q];
                pv[q] = keep ? val : 0.f;
                rsum += pv[q];
              }
              *(uint2*)(Ps + n * PSS + ol) = make_uint2(pack2<F16>(pv[0], pv[1]), pack2<F16>(pv[2], pv[3]));
            }
            if (!IS_DV && own) {
              const float tot = rsum + __shfl_xor(rsum, 32);
              if (h == 0) rows[(2 * kh + kb) * 128 + n] = tot;  // blocks above the diagonal publish zero
            }
          }
          // Out^T += Xw^T P over the 64 source positions of the half: two slabs of 32
#pragma unroll
          for (int vi = 0; vi < 2; ++vi) {
            __syncthreads();
            const int le = opaque(lane);
            const int r = le & 31, h = le >> 5;
            const int q16 = (le >> 4) & 1, i16 = le & 15;
            const int krow = 8 * h + (i16 >> 2), ncol = 16 * q16 + 4 * (i16 & 3);
            const uint16_t* const slab = ((kh + vi) & 1) ? Ring0 : Ring1;
#pragma unroll
            for (int k16 = 0; k16 < 2; ++k16) {
              Frag A[4], B[2];
#pragma unroll
              for (int mb = 0; mb < 4; ++mb) {
                const uint16_t* pp = slab + (16 * k16 + krow) * VS + (128 * ci + 32 * mb + ncol);
                A[mb].d[0] = lds_read_tr16(pp);
                A[mb].d[1] = lds_read_tr16(pp + 4 * VS);
              }
#pragma unroll
              for (int nb = 0; nb < 2; ++nb)
                B[nb].u = *(const uint4*)(Ps + (64 * pi + 32 * nb + r) * PSS + 32 * vi + 16 * k16 + 8 * h);
#pragma unroll
              for (int mb = 0; mb < 4; ++mb)
#pragma unroll
                for (int nb = 0; nb < 2; ++nb) mfma32<F16>(acc[mb][nb], A[mb], B[nb]);
            }
            if constexpr (NORM) {
              // ---- sums over this wave's 128 columns of every row, from the finished accumulators
              if (own && kh == 1 && vi == 1) {
#pragma unroll
                for (int nb = 0; nb < 2; ++nb) {
                  float s1 = 0.f, s2 = 0.f;
#pragma unroll
                  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                      const float x = acc[mb][nb][i];
                      s1 += x;
                      s2 = __builtin_fmaf(x, x, s2);
                    }
                  s1 += __shfl_xor(s1, 32);
                  s2 += __shfl_xor(s2, 32);
                  if (h == 0) {
                    nst[ci * 256 + 64 * pi + 32 * nb + r] = s1;
                    nst[ci * 256 + 128 + 64 * pi + 32 * nb + r] = s2;
                  }
                }
              }
            }
            // ---- forward: denominators, once all row sums of the own chunk are there (it is the last source chunk)
            if (!IS_DV && own && kh == 1 && vi == 1) {
              const int td = opaque(tid);
              const int t = td >> 2;
              if ((td & 3) == 0) {
                float nmax = 1.f, iv = 1.f;
                const float mcr = mcv[t];
                if (a.use_nrow) {
                  float den = denq[t];
#pragma unroll
                  for (int b4 = 0; b4 < 4; ++b4) den += rows[b4 * 128 + t];
                  const float floor_v = a.sig_gate ? 1.f : __expf(-mcr);
                  nmax = fmaxf(fabsf(den), floor_v);
                  iv = 1.f / (nmax + a.eps);
                }
                inv[t] = iv;
                if (it.ch == 0) {
                  a.nrow_out[gofs + t] = nmax;
                  const size_t tg = (size_t)bh * S + (size_t)c * kChunk + t;
                  if (a.n_out != nullptr) a.n_out[tg] = nmax;
                  if (a.m_out != nullptr) a.m_out[tg] = mcr;
                }
              }
            }
          }
        }
      }
      prev = it;
      have_prev = true;
    }
    if (have_prev) {
      __syncthreads();
      HV_EPILOGUE(0, 0, 4, Ring0 + wave * (32 * 136))
      __syncthreads();
      HV_EPILOGUE(1, 0, 4, Ring0 + wave * (32 * 136))
    }
#undef HV_EPILOGUE
  }
}

bool stream_hv_supported(const ParHvArgs& a) {
  // with the fused head norm a work item must hold complete rows: one group of 512 value columns
  const bool norm_ok = a.head_norm == 0 || (a.DHHV == 512 && a.norm_mean != nullptr && a.norm_rstd != nullptr);
  return a.DHQK == 256 && a.DHHV % 512 == 0 && a.S % kChunk == 0 && norm_ok;
}

namespace {
int device_cu_count() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
    cached[dev] = n;
  }
  return cached[dev];
}

template <bool IS_DV, bool F16, bool NORM = false>
const char* launch_stream_hv_t(const ParHvArgs& a, int BH, hipStream_t stream) {
  constexpr int QS = 256 + 8, PSS = 72, SLOT = 64 * QS;
  const size_t smem = (size_t)(128 * QS + 128 * PSS + 2 * SLOT) * 2 +
                      (size_t)(4 * 128 + 128 + 256 + 64 + 64 + 128 + 128 + (NORM ? 8 * 128 : 0)) * 4;
  const long long n_items = (long long)BH * a.NC * (a.DHHV / 512);
  if (n_items >= (1ll << 31)) return "stream_hv: too many work items";
  if ((size_t)a.S * (size_t)a.DHHV * 2 >= ((size_t)1 << 32)) return "stream_hv: one (batch, head) slab of an input exceeds 4 GiB";
  const int cus = device_cu_count();
  if (cus <= 0) return "stream_hv: cannot read the number of compute units";
  int G = (int)(n_items < cus ? n_items : cus);
  if (G >= 8) G -= G % 8;
  const int n_rounds = (int)((n_items + G - 1) / G);
  if (hipFuncSetAttribute((const void*)stream_hv_kernel<IS_DV, F16, NORM>, hipFuncAttributeMaxDynamicSharedMemorySize,
                          (int)smem) != hipSuccess)
    return "stream_hv: cannot raise the dynamic LDS limit";
  hipLaunchKernelGGL((stream_hv_kernel<IS_DV, F16, NORM>), dim3(G), dim3(768), smem, stream, a, (int)n_items, n_rounds);
  return nullptr;
}
}  // namespace

const char* launch_stream_hv(const ParHvArgs& a, int BH, bool is_dv, hipStream_t stream) {
  if (!stream_hv_supported(a))
    return "stream_hv: unsupported shape (needs DHQK = 256, DHHV % 512 == 0, S % 128 == 0; with a head norm DHHV = 512)";
  if (a.stride < 1 || a.stride > kMaxStateStride) return "stream_hv: state stride out of range";
  if (is_dv) return a.f16 ? launch_stream_hv_t<true, true>(a, BH, stream) : launch_stream_hv_t<true, false>(a, BH, stream);
  if (a.head_norm != 0)
    return a.f16 ? launch_stream_hv_t<false, true, true>(a, BH, stream) : launch_stream_hv_t<false, false, true>(a, BH, stream);
  return a.f16 ? launch_stream_hv_t<false, true>(a, BH, stream) : launch_stream_hv_t<false, false>(a, BH, stream);
}

}  // namespace mlstm

