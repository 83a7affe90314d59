// Streaming form of the chunk-parallel backward kernels whose output tile spans the query/key head dimension (dQ and
// dK): the same arithmetic as par_qk.hip (see there for the formulas and the state-stride algebra), organised like
// stream_hv.hip around HBM bandwidth and the LDS read port.
//
//   * One PERSISTENT workgroup per CU (twelve waves) walks its share of the work items; an item is one gradient (dQ or
//     dK) of one chunk of 128 positions x all 256 head-dimension rows of one (batch, head).  The two items of a chunk
//     are neighbours in the item order, so the V and dH rows both stream meet in the L2.
//   * Four PRODUCER waves move data only: every operand is cut into slabs of 32 KB (the state for 64 value columns as
//     stored fragments; 128 Xn + 128 Xo rows x 64 value columns; 64 Z rows x 256 head-dim entries), two slabs are on
//     their way in registers at any time, across item boundaries.  Eight CONSUMER waves own 64 head-dim rows x 64
//     positions of the output (64 accumulator registers) and two 32 x 32 score blocks each; they read operand
//     fragments from LDS, multiply, gate, and write the output rows and the row dots straight from the accumulators.
//   * One barrier per slab; the ring has three slots because the inter-chunk product of a 64-column step needs the
//     state slab and the row slab of that step together (the row slab comes first and feeds the score blocks alone).
//     Both roles walk the same item list with the same number of steps per item (18 for the own chunk, 10 for every
//     further source chunk), so they pass the same number of barriers by construction.
//
// Step sequence of an item (the own chunk first, then the other source chunks of its stride window):
//   own chunk:     8 x [ row slab w (scores += Xo Xn^T), state slab w (Out^T += State Xn^T) ], gate -> P,
//                  2 x Z slab (Out^T += Z^T P)
//   further chunk: 8 x row slab (scores), gate -> P, 2 x Z slab
//   then the row dots sum_d x Out (x = q for dQ, k for dK) and the output rows leave from the accumulators.
// Supported: DHQK = 256, DHHV a multiple of 128, S a multiple of 128; everything else runs par_qk.hip.
#include "common.h"
#include "kernels.h"

namespace mlstm {
namespace {

struct QkItem {
  int bh, c, dk;       // (batch * head), chunk, gradient (0 dQ, 1 dK)
  int slot;            // kept boundary state the chunk uses
  int sc_lo, sc_hi;    // source chunks of the stride window
};

__device__ __forceinline__ bool qk_decode(QkItem& it, int round, int vid, int G, int n_items, int NC, int stride) {
  const int rot = (vid + round) % G;
  const long long idx = (long long)round * G + rot;
  if (idx >= n_items) return false;
  const int i = (int)idx;
  it.dk = i & 1;
  const int rest = i >> 1;
  it.c = rest % NC;
  it.bh = rest / NC;
  it.slot = it.c / stride;
  if (it.dk) {
    it.sc_lo = it.c;
    it.sc_hi = min(it.slot * stride + stride - 1, NC - 1);
  } else {
    it.sc_lo = it.slot * stride;
    it.sc_hi = it.c;
  }
  return true;
}

constexpr float kQkLog2e = 1.4426950408889634f;

}  // namespace

template <bool F16>
__global__ __launch_bounds__(768) void stream_qk_kernel(ParQkArgs a, int n_items, int n_rounds) {
  constexpr int DHQK = 256;
  constexpr int XS = 64 + 8;     // row slab: [128 Xn rows | 128 Xo rows] x 64 value columns
  constexpr int ZS = DHQK + 32;  // Z slab: 64 rows x 256 head-dim entries (rows 64 bytes apart in the banks)
  constexpr int PS = 128 + 8;    // gated score block P[n][o]: 128 positions x 128 source positions
  constexpr int SLOT = 64 * ZS;  // elements per ring slot (36 KB: the largest slab kind)
  constexpr int ND = DHQK / 16;
  static_assert(256 * XS <= SLOT && 16384 <= SLOT, "every slab kind fits a ring slot");
  extern __shared__ __align__(16) unsigned char smem_raw[];
  uint16_t* const Ring = (uint16_t*)smem_raw;     // [3][SLOT]
  uint16_t* const Ps = Ring + 3 * SLOT;
  float* const ovec = (float*)(Ps + 128 * PS);    // [128] gate vector of the source chunk: w_j (dQ) / u_t (dK)
  float* const orho = ovec + 128;                 // [128] dK: rho_t of the source chunk (dQ: ones)
  float* const red = orho + 128;                  // [4][128] row-dot partials of the previous item, per 64-row block

  const int lane = threadIdx.x & 63;
  const int wave_all = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int G = gridDim.x;
  int vid = blockIdx.x;
  if (G % 8 == 0) vid = (vid % 8) * (G / 8) + vid / 8;  // consecutive ids share an XCD (and its L2)
  const int NC = a.NC, S = a.S, DHHV = a.DHHV, stride = a.stride;
  const int NW = DHHV / 64;  // 64-column steps over the value dimension
  const size_t Sp = (size_t)NC * kChunk;
  const int NCS = (NC + stride - 1) / stride;

  if (wave_all >= 8) {
    // =========================================================================================== producer waves
    // Load step L (counted over all items of this workgroup) uses register set L & 1 and ring slot L % 3.  Handling it
    // means: pass barrier L - 3, write slab L - 2 from the register set to LDS, request slab L into the set.  The
    // destination in LDS travels with the data: byte offset of the thread's first piece | piece distance code << 20
    // (0: 4096 bytes, 1: 4608 bytes) | gate-vector flag << 22 | reciprocal-of-the-normaliser flag << 23.
    const int p = (wave_all - 8) * 64 + lane;  // 0 .. 255: every thread moves eight 16-byte pieces of every slab
    u32x4 fd0[8], fd1[8];
    uint32_t fw0 = 0, fw1 = 0;
    float fa0[2], fa1[2];
    int L = 0;
    uint32_t ring_slot = 0;  // L % 3
#define QK_STORE(E)                                                                                                  \
  {                                                                                                                  \
    const uint32_t w_ = fw##E;                                                                                       \
    const uint32_t step_ = __builtin_amdgcn_readfirstlane((int)((w_ >> 20) & 1)) ? 4608u : 4096u;                    \
    const uint32_t d0_ = w_ & 0xFFFFFu;                                                                              \
    _Pragma("unroll") for (int i_ = 0; i_ < 8; ++i_) *(u32x4*)(smem_raw + d0_ + i_ * step_) = fd##E[i_];             \
    if (__builtin_amdgcn_readfirstlane((int)((w_ >> 22) & 1)) && p < 128) {                                          \
      ovec[p] = fa##E[0];                                                                                 \
      orho[p] = __builtin_amdgcn_readfirstlane((int)((w_ >> 23) & 1)) ? 1.f / (fa##E[1] + a.eps) : 1.f;              \
    }                                                                                                                \
  }
    // one step: bA_/gA_/sA_ base, first byte offset and piece distance of pieces 0..3, bB_/gB_/sB_ of pieces 4..7
    // (a row slab has two sources); dst_ destination word without the slot; gi_ gate-vector index that rides along
#define QK_PROC(E, bA_, gA_, sA_, bB_, gB_, sB_, dst_, gi_)                                                          \
  {                                                                                                                  \
    if (L >= 3) __syncthreads();                                                                                           \
    /* piece by piece: the old content of a register goes to LDS, then the register is requested anew, so that the */ \
    /* LDS port and the vector-memory path of the CU work side by side instead of one after the other */             \
    const uint32_t w_ = fw##E;                                                                                       \
    const uint32_t step_ = __builtin_amdgcn_readfirstlane((int)((w_ >> 20) & 1)) ? 4608u : 4096u;                    \
    const uint32_t d0_ = w_ & 0xFFFFFu;                                                                              \
    const bool st_ = L >= 2;                                                                                         \
    if (st_ && __builtin_amdgcn_readfirstlane((int)((w_ >> 22) & 1)) && p < 128) {                                   \
      ovec[p] = fa##E[0];                                                                                 \
      orho[p] = __builtin_amdgcn_readfirstlane((int)((w_ >> 23) & 1)) ? 1.f / (fa##E[1] + a.eps) : 1.f;              \
    }                                                                                                                \
    fa##E[0] = ov_src[gi_];                                                                                          \
    fa##E[1] = rho_src[gi_];                                                                                         \
    _Pragma("unroll") for (int i_ = 0; i_ < 4; ++i_) {                                                               \
      if (st_) *(u32x4*)(smem_raw + d0_ + i_ * step_) = fd##E[i_];                                                   \
      fd##E[i_] = *(const u32x4*)((bA_) + ((gA_) + i_ * (sA_)));                                                     \
    }                                                                                                                \
    _Pragma("unroll") for (int i_ = 0; i_ < 4; ++i_) {                                                               \
      if (st_) *(u32x4*)(smem_raw + d0_ + (4 + i_) * step_) = fd##E[4 + i_];                                         \
      fd##E[4 + i_] = *(const u32x4*)((bB_) + ((gB_) + i_ * (sB_)));                                                 \
    }                                                                                                                \
    fw##E = (dst_) + ring_slot * (SLOT * 2);                                                                         \
    ring_slot = ring_slot == 2 ? 0 : ring_slot + 1;                                                                  \
    ++L;                                                                                                             \
  }
    QkItem it;
    for (int rd = 0; rd < n_rounds; ++rd) {
      if (!qk_decode(it, rd, vid, G, n_items, NC, stride)) continue;
      const uint32_t pl = (uint32_t)opaque(p);
      const char* const Xn_b = (const char*)(it.dk ? a.V : a.dH) + (size_t)it.bh * S * DHHV * 2;
      const char* const Xo_b = (const char*)(it.dk ? a.dH : a.V) + (size_t)it.bh * S * DHHV * 2;
      const char* const Z_b = (const char*)(it.dk ? a.Q : a.K) + (size_t)it.bh * S * DHQK * 2;
      const char* const St_b = (const char*)(it.dk ? a.states2 : a.states) +
                               ((size_t)it.bh * NCS + it.slot) * (size_t)(DHHV / 32) * ND * 1024;
      const float* const ov_src = it.dk ? a.g.u : a.g.w;
      const bool with_rho = it.dk && a.use_nrow;  // dK: rho_t of the source rows rides along (dQ: ones)
      const float* const rho_src = with_rho ? a.nrow : ov_src;
      const size_t hofs = (size_t)it.bh * Sp;
      // row slab: piece (row, pc) = (pl / 8 + 32 i, pl % 8), 128 bytes per row and source
      const uint32_t xrow = pl >> 3, xpc = pl & 7;
      const uint32_t xdst = (xrow * (XS * 2) + xpc * 16) | (1u << 20);
      const uint32_t xn0 = ((uint32_t)(it.c * kChunk) + xrow) * (uint32_t)(DHHV * 2) + xpc * 16;
      const uint32_t xstep = 32 * (uint32_t)DHHV * 2;
      // state slab: 32 KB of stored fragments, contiguous in memory; lanes 32..63 of every fragment are stored 4
      // slots off so that the two lane halves a transposing read touches together fall on different LDS banks
      const uint32_t cdst = (pl ^ (((pl >> 5) & 1) << 2)) * 16;
      // Z slab: piece (row, pc) = (pl / 32 + 8 i, pl % 32), 512 bytes per row
      const uint32_t zrow = pl >> 5, zpc = pl & 31;
      const uint32_t zdst = (zrow * (ZS * 2) + zpc * 16) | (1u << 20);
      for (int k = 0; k <= it.sc_hi - it.sc_lo; ++k) {
        // the own chunk first, then the others in ascending order
        const int sc = k == 0 ? it.c : (it.sc_lo + k - 1 < it.c ? it.sc_lo + k - 1 : it.sc_lo + k);
        const bool own = k == 0;
        const uint32_t xo0 = ((uint32_t)(sc * kChunk) + xrow) * (uint32_t)(DHHV * 2) + xpc * 16;
        const size_t gi = hofs + (size_t)sc * kChunk + (pl & 127);
        for (int ws = 0; ws < NW; ++ws) {
          const uint32_t flag = ws == 0 ? ((1u << 22) | (with_rho ? 1u << 23 : 0u)) : 0u;
          if (own) {
            QK_PROC(0, Xn_b, xn0 + ws * 128, xstep, Xo_b, xo0 + ws * 128, xstep, xdst | flag, gi)
            QK_PROC(1, St_b, (uint32_t)ws * 32768 + pl * 16, 4096, St_b, (uint32_t)ws * 32768 + 16384 + pl * 16, 4096, cdst, gi)
          } else {
            QK_PROC(0, Xn_b, xn0 + ws * 128, xstep, Xo_b, xo0 + ws * 128, xstep, xdst | flag, gi)
            ++ws;
            QK_PROC(1, Xn_b, xn0 + ws * 128, xstep, Xo_b, xo0 + ws * 128, xstep, xdst, gi)
          }
        }
        const uint32_t z0 = ((uint32_t)(sc * kChunk) + zrow) * (DHQK * 2) + zpc * 16;
        QK_PROC(0, Z_b, z0, 8 * DHQK * 2, Z_b, z0 + 32 * DHQK * 2, 8 * DHQK * 2, zdst, gi)
        QK_PROC(1, Z_b, z0 + 64 * DHQK * 2, 8 * DHQK * 2, Z_b, z0 + 96 * DHQK * 2, 8 * DHQK * 2, zdst, gi)
      }
    }
    // ---- drain: the last two slabs go to LDS, then the barriers of the consumers' last steps and of the final row dots
    if (L > 0) {
      if (L >= 3) __syncthreads();
      QK_STORE(0)
      __syncthreads();
      QK_STORE(1)
      __syncthreads();
      __syncthreads();
    }
#undef QK_PROC
#undef QK_STORE
  } else {
    // =========================================================================================== consumer waves
    const int wave = wave_all;
    const int tid = wave * 64 + lane;
    const int di = wave & 3, ni = wave >> 2;   // output role: head-dim rows 64 di .., positions 64 ni ..
    const int nbk = wave & 3, oq = wave >> 2;  // score role: position block nbk, source blocks 2 oq and 2 oq + 1
    f32x16 acc[2][2], sacc[2];
    QkItem it, prev;
    prev = QkItem{0, 0, 0, 0, 0, 0};
    bool have_prev = false;
    uint32_t slot = 0;  // ring slot of the next slab (step % 3)
    auto next_slot = [&]() {
      const uint32_t s = slot;
      slot = slot == 2 ? 0 : slot + 1;
      return s;
    };
    // row dots of the previous item: the four 64-row blocks' partials meet in LDS, 128 threads add them up
    auto finish_rowdots = [&]() {
      if (have_prev && tid < 128) {
        const float dot = (red[tid] + red[128 + tid]) + (red[256 + tid] + red[384 + tid]);
        (prev.dk ? a.rowdot2 : a.rowdot)[(size_t)prev.bh * Sp + (size_t)prev.c * kChunk + tid] = dot;
      }
    };
    for (int rd = 0; rd < n_rounds; ++rd) {
      if (!qk_decode(it, rd, vid, G, n_items, NC, stride)) continue;
      const int bh = it.bh, c = it.c;
      const bool dk = it.dk != 0;
      const size_t hofs = (size_t)bh * Sp, gofs = hofs + (size_t)c * kChunk;
      const float* graw = a.g.graw + (size_t)bh * NC;
      const float* mst = a.g.mstates + (size_t)bh * (NC + 1);
      // ---- per-item vectors (requested now, used after the first pass over the value columns)
      float csr[2], nv, nrho = 1.f;
      {
        const int r = opaque(lane) & 31;
        float gsum = 0.f, xs = 1.f;
        if (dk) {
          for (int x = c + 1; x <= it.sc_hi; ++x) gsum += graw[x];
          if (it.sc_hi > c) xs = __expf(gsum + mst[c + 1] - mst[it.sc_hi + 1]);
        } else {
          for (int x = it.sc_lo; x < c; ++x) gsum += graw[x];
          if (it.sc_lo < c) xs = __expf(gsum + mst[it.sc_lo] - mst[c]);
        }
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
          const size_t gi = gofs + 64 * ni + 32 * nb + r;
          const float rh = a.use_nrow ? 1.f / (a.nrow[gi] + a.eps) : 1.f;
          csr[nb] = (dk ? a.g.abar[gi] : a.g.bbar[gi] * a.qk_scale * rh) * xs;
        }
        const size_t gn = gofs + 32 * nbk + r;
        nv = (dk ? a.g.w : a.g.u)[gn];
        if (!dk && a.use_nrow) nrho = 1.f / (a.nrow[gn] + a.eps);
      }
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.f;
      const int nsc = it.sc_hi - it.sc_lo + 1;
      uint2 xr[2][2][4];  // the x rows of the row dots in accumulator layout, requested during the last source chunk

      // One row slab: score blocks (2 oq + kk, nbk) += Xo Xn^T over its 64 value columns.  LIVE_: in the own chunk the
      // causal mask empties the blocks with o > n (dQ) or o < n (dK); a wave whose two blocks are both empty skips the
      // multiplications (its rows of P stay zero).
#define QK_XSTEP(LIVE_)                                                                                              \
  __syncthreads();                                                                                                   \
  const uint16_t* const Xn = Ring + next_slot() * SLOT;                                                              \
  {                                                                                                                  \
    const uint16_t* const Xo = Xn + 128 * XS;                                                                        \
    const int le = opaque(lane);                                                                                     \
    const int r = le & 31, h = le >> 5;                                                                              \
    if (LIVE_) {                                                                                                     \
      _Pragma("unroll") for (int k16 = 0; k16 < 4; ++k16) {                                                          \
        Frag B, A[2];                                                                                                \
        B.u = *(const uint4*)(Xn + (32 * nbk + r) * XS + 16 * k16 + 8 * h);                                          \
        _Pragma("unroll") for (int kk = 0; kk < 2; ++kk)                                                             \
          A[kk].u = *(const uint4*)(Xo + (32 * (2 * oq + kk) + r) * XS + 16 * k16 + 8 * h);                          \
        _Pragma("unroll") for (int kk = 0; kk < 2; ++kk) mfma32<F16>(sacc[kk], A[kk], B);                            \
      }                                                                                                              \
    }                                                                                                                \
  }
      // Gate the score blocks: P[o][n] = scores * exp(u_t - w_j + G) / sqrt(DHQK) * rho_t (own chunk: masked), stored
      // as Ps[n][o]; sc_: source chunk, OWN_: it is the own one
#define QK_GATE(sc_, OWN_)                                                                                           \
  {                                                                                                                  \
    float gs = 0.f; /* decay between the two chunks */                                                               \
    for (int x = (dk ? c : (sc_)); x < (dk ? (sc_) : c); ++x) gs += graw[x];                                         \
    const float sgn = dk ? -1.f : 1.f;                                                                               \
    const float un = nv + sgn * gs;                                                                                  \
    const float lq = __log2f(a.qk_scale);                                                                            \
    const int le = opaque(lane);                                                                                     \
    const int r = le & 31, h = le >> 5;                                                                              \
    const int n = 32 * nbk + r;                                                                                      \
    _Pragma("unroll") for (int kk = 0; kk < 2; ++kk) _Pragma("unroll") for (int g4 = 0; g4 < 4; ++g4) {              \
      const int o0 = 32 * (2 * oq + kk) + 8 * g4 + 4 * h;                                                            \
      const float4 xo = *(const float4*)(ovec + o0);                                                                 \
      const float4 ro = *(const float4*)(orho + o0);                                                                 \
      const float xov[4] = {xo.x, xo.y, xo.z, xo.w};                                                                 \
      const float rov[4] = {ro.x, ro.y, ro.z, ro.w};                                                                 \
      float pv[4];                                                                                                   \
      _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                                                \
        const float e2 = __builtin_amdgcn_exp2f(__builtin_fmaf(sgn * (un - xov[q]), kQkLog2e, lq));                  \
        const bool keep = !(OWN_) || (dk ? (n <= o0 + q) : (o0 + q <= n));                                           \
        const float val = sacc[kk][4 * g4 + q] * e2 * (nrho * rov[q]);                                               \
        pv[q] = keep ? val : 0.f;                                                                                    \
      }                                                                                                              \
      *(uint2*)(Ps + n * PS + o0) = make_uint2(pack2<F16>(pv[0], pv[1]), pack2<F16>(pv[2], pv[3]));                  \
    }                                                                                                                \
  }
      // Out^T += Z^T P over the 128 source positions, 64 per slab; LAST_: the x rows of the row dots are requested
      // with the first slab
#define QK_PASS2(LAST_)                                                                                              \
  _Pragma("unroll") for (int zs = 0; zs < 2; ++zs) {                                                                 \
    __syncthreads();                                                                                                 \
    const uint16_t* const Zs = Ring + next_slot() * SLOT;                                                            \
    const int le = opaque(lane);                                                                                     \
    const int r = le & 31, h = le >> 5;                                                                              \
    const int q16 = (le >> 4) & 1, i16 = le & 15;                                                                    \
    const int krow = 8 * h + (i16 >> 2), ncol = 16 * q16 + 4 * (i16 & 3);                                            \
    if ((LAST_) && zs == 0) {                                                                                        \
      const uint16_t* Rg = (dk ? a.K : a.Q) + ((size_t)bh * S + (size_t)c * kChunk) * DHQK;                          \
      _Pragma("unroll") for (int mb = 0; mb < 2; ++mb) _Pragma("unroll") for (int nb = 0; nb < 2; ++nb)              \
        _Pragma("unroll") for (int g4 = 0; g4 < 4; ++g4)                                                             \
          xr[mb][nb][g4] = *(const uint2*)(Rg + (size_t)(64 * ni + 32 * nb + r) * DHQK + 64 * di + 32 * mb + 8 * g4 + 4 * h); \
    }                                                                                                                \
    _Pragma("unroll") for (int k16 = 0; k16 < 4; ++k16) {                                                            \
      Frag A[2], B[2];                                                                                               \
      _Pragma("unroll") for (int mb = 0; mb < 2; ++mb) {                                                             \
        const uint16_t* pp = Zs + (16 * k16 + krow) * ZS + (64 * di + 32 * mb + ncol);                               \
        A[mb].d[0] = lds_read_tr16(pp);                                                                              \
        A[mb].d[1] = lds_read_tr16(pp + 4 * ZS);                                                                     \
      }                                                                                                              \
      _Pragma("unroll") for (int nb = 0; nb < 2; ++nb)                                                               \
        B[nb].u = *(const uint4*)(Ps + (64 * ni + 32 * nb + r) * PS + 64 * zs + 16 * k16 + 8 * h);                   \
      _Pragma("unroll") for (int mb = 0; mb < 2; ++mb) _Pragma("unroll") for (int nb = 0; nb < 2; ++nb)              \
        mfma32<F16>(acc[mb][nb], A[mb], B[nb]);                                                                      \
    }                                                                                                                \
  }
#define QK_ZERO_SCORES                                                                                               \
  _Pragma("unroll") for (int kk = 0; kk < 2; ++kk) _Pragma("unroll") for (int i = 0; i < 16; ++i) sacc[kk][i] = 0.f;

      // ---- the own chunk: one pass over the value columns, 64 at a time, feeds the score blocks (row slab) and the
      // inter-chunk product (state slab of the same columns)
      {
        const bool live = dk ? (2 * oq + 1 >= nbk) : (2 * oq <= nbk);
        QK_ZERO_SCORES
        for (int ws = 0; ws < NW; ++ws) {
          QK_XSTEP(live)
          if (ws == 0) finish_rowdots();
          // Out^T += State Xn^T.  The stored fragments (made for a contraction over the head dimension) are read with
          // the transposing LDS read: lane i16 of a 16-lane block addresses value column k0 + i16 / 4 and the 4
          // consecutive head-dim rows n0 + 4 (i16 % 4) .. + 3
          __syncthreads();
          const uint16_t* const Cf = Ring + next_slot() * SLOT;
          const int le = opaque(lane);
          const int r = le & 31, h = le >> 5;
          const int q16 = (le >> 4) & 1, i16 = le & 15;
          const int d_grp = i16 & 3;
          const int h_src = d_grp & 1, a_src = d_grp >> 1;
#pragma unroll
          for (int sub = 0; sub < 2; ++sub)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
              Frag A[2], B[2];
#pragma unroll
              for (int nb = 0; nb < 2; ++nb)
                B[nb].u = *(const uint4*)(Xn + (64 * ni + 32 * nb + r) * XS + 32 * sub + 16 * ks + 8 * h);
              const int wrow = 16 * ks + 8 * h + (i16 >> 2);  // value column inside the 32-column half (first read)
#pragma unroll
              for (int mb = 0; mb < 2; ++mb) {
                const int ds_l = (64 * di + 32 * mb + 16 * q16) / 16;
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                  const int wr = wrow + 4 * half;
                  const int slot_l = (32 * h_src + wr) ^ (h_src << 2);
                  const unsigned char* pp = (const unsigned char*)Cf + sub * 16384 + ((size_t)ds_l * 64 + slot_l) * 16 + 8 * a_src;
                  A[mb].d[half] = lds_read_tr16(pp);
                }
              }
#pragma unroll
              for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                for (int nb = 0; nb < 2; ++nb) mfma32<F16>(acc[mb][nb], A[mb], B[nb]);
            }
        }
        // column scale of the inter-chunk part (kept apart from the matrix instructions around it)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
          for (int mb = 0; mb < 2; ++mb) acc[mb][nb] *= csr[nb];
        __builtin_amdgcn_sched_barrier(0);
        QK_GATE(c, true)
        QK_PASS2(nsc == 1)
      }
      // ---- the other source chunks of the stride window, in ascending order: scores, gate, Out^T += Z^T P
      for (int k = 1; k < nsc; ++k) {
        const int sc = it.sc_lo + k - 1 < c ? it.sc_lo + k - 1 : it.sc_lo + k;
        QK_ZERO_SCORES
        for (int ws = 0; ws < NW; ++ws) {
          QK_XSTEP(true)
        }
        QK_GATE(sc, false)
        QK_PASS2(k == nsc - 1)
      }
#undef QK_XSTEP
#undef QK_GATE
#undef QK_PASS2
#undef QK_ZERO_SCORES
      {
        // ---- row dots sum_d x[n][d] * Out[n][d] from the fp32 accumulators (they feed a suffix sum over the whole
        // sequence, where the rounding noise of 16-bit outputs would add up), and the output rows, rounded, straight
        // from the accumulators: 16 contiguous bytes per row and lane pair
        const int le = opaque(lane);
        const int r = le & 31, h = le >> 5;
        uint16_t* const Og = (dk ? a.Out2 : a.Out) + ((size_t)bh * S + (size_t)c * kChunk) * DHQK;
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
          float part = 0.f;
#pragma unroll
          for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
              const uint2 xv = xr[mb][nb][g4];
              part += acc[mb][nb][4 * g4 + 0] * lo2<F16>(xv.x);
              part += acc[mb][nb][4 * g4 + 1] * hi2<F16>(xv.x);
              part += acc[mb][nb][4 * g4 + 2] * lo2<F16>(xv.y);
              part += acc[mb][nb][4 * g4 + 3] * hi2<F16>(xv.y);
              *(uint2*)(Og + (size_t)(64 * ni + 32 * nb + r) * DHQK + 64 * di + 32 * mb + 8 * g4 + 4 * h) =
                  make_uint2(pack2<F16>(acc[mb][nb][4 * g4 + 0], acc[mb][nb][4 * g4 + 1]),
                             pack2<F16>(acc[mb][nb][4 * g4 + 2], acc[mb][nb][4 * g4 + 3]));
            }
          part += __shfl_xor(part, 32);
          if (h == 0) red[di * 128 + 64 * ni + 32 * nb + r] = part;
        }
      }
      prev = it;
      have_prev = true;
    }
    if (have_prev) {
      __syncthreads();
      finish_rowdots();
    }
  }
}

bool stream_qk_supported(const ParQkArgs& a) { return a.DHQK == 256 && a.DHHV % 128 == 0 && a.S % kChunk == 0; }

namespace {
int qk_device_cu_count() {
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

template <bool F16>
const char* launch_stream_qk_t(const ParQkArgs& a, int BH, hipStream_t stream) {
  constexpr int ZS = 256 + 32, PS = 128 + 8, SLOT = 64 * ZS;
  const size_t smem = (size_t)(3 * SLOT + 128 * PS) * 2 + (size_t)(128 + 128 + 4 * 128) * 4;
  const long long n_items = (long long)BH * a.NC * 2;
  if (n_items >= (1ll << 31)) return "stream_qk: too many work items";
  if ((size_t)a.S * (size_t)(a.DHHV > a.DHQK ? a.DHHV : a.DHQK) * 2 >= ((size_t)1 << 32))
    return "stream_qk: one (batch, head) slab of an input exceeds 4 GiB";
  const int cus = qk_device_cu_count();
  if (cus <= 0) return "stream_qk: cannot read the number of compute units";
  int G = (int)(n_items < cus ? n_items : cus);
  if (G >= 8) G -= G % 8;
  const int n_rounds = (int)((n_items + G - 1) / G);
  if (hipFuncSetAttribute((const void*)stream_qk_kernel<F16>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
    return "stream_qk: cannot raise the dynamic LDS limit";
  hipLaunchKernelGGL((stream_qk_kernel<F16>), dim3(G), dim3(768), smem, stream, a, (int)n_items, n_rounds);
  return nullptr;
}
}  // namespace

const char* launch_stream_qk(const ParQkArgs& a, int BH, hipStream_t stream) {
  if (!stream_qk_supported(a)) return "stream_qk: unsupported shape (needs DHQK = 256, DHHV % 128 == 0, S % 128 == 0)";
  if (a.states2 == nullptr || a.Out2 == nullptr || a.rowdot2 == nullptr) return "stream_qk: the dK operands are missing";
  if (a.stride < 1 || a.stride > kMaxStateStride) return "stream_qk: state stride out of range";
  return a.f16 ? launch_stream_qk_t<true>(a, BH, stream) : launch_stream_qk_t<false>(a, BH, stream);
}

}  // namespace mlstm

