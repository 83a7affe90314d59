// dQ and dK of the chunkwise backward for the default state stride of 2, organised around the window of two chunks
// that share a kept state: the same arithmetic as par_qk.hip (see there for the formulas and the state-stride
// algebra), arranged so that every operand passes through a CU as few times as the register file allows and the
// score blocks are computed once for both gradients.
//
// With c0 = 2s, c1 = 2s + 1 the two chunks of window s (256 positions, t and j counted over the window), C the state
// kept before c0 and dC the state kept after c1:
//   P[t][j]   = exp(u_t - w_j + G) / sqrt(DHQK) * rho_t * (dH_t . v_j)   for j <= t   (G = decay of c0 when t is in
//               c1 and j in c0, else 0): a lower triangle of 8 x 8 blocks of 32 x 32, 36 blocks, kept in LDS as bf16
//   dQ[t][:]  = csq_t * (C dH_t)  + sum_j P[t][j] k_j
//   dK[j][:]  = csk_j * (dC v_j)  + sum_t P[t][j] q_t
//
//   * One PERSISTENT workgroup per CU (twelve waves) walks its share of the windows.  Four PRODUCER waves move data
//     only, in slabs of 32 KB through a FIFO of two register sets into a ring of two LDS slots; eight CONSUMER waves
//     read operand fragments from LDS, multiply, gate and write the results.  One barrier per slab.
//   * Three phases per window, all with a static step structure (NV = DHHV / 32):
//       S  NV steps  [dH rows x 32 value columns | V rows x 32 value columns]      scores of all 36 blocks, then gating
//       Q  NV steps  [C fragments of 32 value columns | dH rows x 32 columns]      Out^T += C dH^T  (256 x 256 tile)
//           4 steps  [64 K rows x 256 head-dim entries]                            Out^T += K^T P^T
//           4 steps  [64 Q rows]                                                   row dots q . dQ; dQ rows leave
//       K  NV steps  [dC fragments | V rows],  4 steps [64 Q rows], 4 steps [64 K rows]   the same for dK (P read
//                                                                                  transposed)
//     A window moves 3 * DHHV + 512 KB through the CU (2048 KB at DHHV = 512) where its four chunk-and-gradient items
//     take 2944 KB in stream_qk.hip, and multiplies every score block once instead of twice.
//   * A consumer wave owns 64 head-dim rows x four 32-position blocks of alternating parity (128 accumulator
//     registers); the causal structure then loads both parities nearly alike.  The q (k) rows of the gate-gradient
//     row dots come through the ring like every other operand (fetched by the consumers themselves they cost a
//     memory latency per handful of positions); the rounded results pass through a private 2 KB staging tile per
//     wave into row order and are stored as full 128-byte lines.
// Supported: state stride 2, DHQK = 256, DHHV a multiple of 64, S a multiple of 256.
#include <type_traits>

#include "common.h"
#include "kernels.h"

namespace mlstm {
namespace {

struct WqItem {
  int bh, win;   // (batch * head), window of two chunks
};

__device__ __forceinline__ bool wq_decode(WqItem& it, int round, int vid, int G, int n_items, int NWIN) {
  const int rot = (vid + round) % G;
  const long long idx = (long long)round * G + rot;
  if (idx >= n_items) return false;
  it.win = (int)idx % NWIN;
  it.bh = (int)idx / NWIN;
  return true;
}

constexpr float kWqLog2e = 1.4426950408889634f;
constexpr int kWqSlot = 32768;                    // bytes per ring slot = per slab
constexpr int kWqPOfs = 2 * kWqSlot;              // P: 36 blocks of 32 x 32 (2 KB each, 64-byte rows, swizzled)
constexpr int kWqVecOfs = kWqPOfs + 36 * 2048;    // u[256], w[256], lqr[256] (fp32)
constexpr int kWqRedOfs = kWqVecOfs + 3 * 1024;   // [4][256] row-dot partials per 64-row block of the head dimension
constexpr int kWqStgOfs = kWqRedOfs + 4 * 1024;   // [8 waves][16 rows][64 elements] staging tiles
constexpr int kWqCsOfs = kWqStgOfs + 8 * 2048;    // [256] column scale of the inter-chunk part of the running phase
constexpr int kWqSmem = kWqCsOfs + 1024;
static_assert(kWqSmem <= 160 * 1024, "LDS budget of one CU");

// the blocks (tb, jb) of the lower triangle a consumer wave computes in phase S: up to five, at most two distinct tb
// (packed: 3 bits tb, 3 bits jb per entry, count in bits 30..32)
__device__ __forceinline__ uint64_t wq_score_blocks(int wave) {
#define E5(t0, j0, t1, j1, t2, j2, t3, j3, t4, j4, n)                                                                \
  ((uint64_t)(t0) | ((uint64_t)(j0) << 3) | ((uint64_t)(t1) << 6) | ((uint64_t)(j1) << 9) | ((uint64_t)(t2) << 12) | \
   ((uint64_t)(j2) << 15) | ((uint64_t)(t3) << 18) | ((uint64_t)(j3) << 21) | ((uint64_t)(t4) << 24) |               \
   ((uint64_t)(j4) << 27) | ((uint64_t)(n) << 30))
  switch (wave) {
    case 0: return E5(7, 0, 7, 1, 7, 2, 7, 3, 0, 0, 5);
    case 1: return E5(7, 4, 7, 5, 7, 6, 7, 7, 7, 7, 4);
    case 2: return E5(6, 0, 6, 1, 6, 2, 6, 3, 6, 3, 4);
    case 3: return E5(6, 4, 6, 5, 6, 6, 1, 0, 1, 1, 5);
    case 4: return E5(5, 0, 5, 1, 5, 2, 5, 3, 5, 3, 4);
    case 5: return E5(5, 4, 5, 5, 2, 0, 2, 1, 2, 2, 5);
    case 6: return E5(4, 0, 4, 1, 4, 2, 4, 3, 4, 4, 5);
    default: return E5(3, 0, 3, 1, 3, 2, 3, 3, 3, 3, 4);
  }
#undef E5
}

// 16-byte-unit swizzle of tiles with 64-byte rows (operand rows of 32 value columns, blocks of P): eight consecutive
// rows read at one unit, and the 4 rows x 2 units patch of a transposing read, both fall on distinct LDS banks
__device__ __forceinline__ int wq_f64(int row) { return (((row >> 1) & 1) << 1) | ((row >> 2) & 1); }

}  // namespace

template <bool F16>
__global__ __launch_bounds__(768) void window_qk_kernel(ParQkArgs a, int n_items, int n_rounds) {
  constexpr int DHQK = 256;
  constexpr int ND = DHQK / 16;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  float* const uvec = (float*)(smem_raw + kWqVecOfs);  // [256] u_t of the window's positions
  float* const wvec = uvec + 256;                      // [256] w_j
  float* const lqr = wvec + 256;                       // [256] log2(rho_t / sqrt(DHQK))
  float* const red = (float*)(smem_raw + kWqRedOfs);
  float* const csv = (float*)(smem_raw + kWqCsOfs);

  const int lane = threadIdx.x & 63;
  const int wave_all = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int G = gridDim.x;
  int vid = blockIdx.x;
  if (G % 8 == 0) vid = (vid % 8) * (G / 8) + vid / 8;  // consecutive ids share an XCD (and its L2)
  const int NC = a.NC, S = a.S, DHHV = a.DHHV;
  const int NV = DHHV / 32;   // steps of 32 value columns (even)
  const int NWIN = NC / 2;
  const size_t Sp = (size_t)NC * kChunk;

  if (wave_all >= 8) {
    // =========================================================================================== producer waves
    // Load step L (counted over all windows of this workgroup) uses register set L & 1 and ring slot L & 1.  Handling
    // it means: pass barrier L - 3, write slab L - 2 from the register set to LDS, request slab L into the set.  The
    // destination in LDS travels with the data: 16-byte-unit offsets of the first piece of either half of the slab
    // (pieces 0..3 and 4..7, 4096 bytes apart inside a half).
    const int p = (wave_all - 8) * 64 + lane;  // 0 .. 255: every thread moves eight 16-byte pieces of every slab
    u32x4 fd0[8], fd1[8];
    uint32_t fw0 = 0, fw1 = 0;
    int L = 0;
#define WQ_STORE(E)                                                                                                  \
  {                                                                                                                  \
    const uint32_t w_ = fw##E;                                                                                       \
    const uint32_t dA_ = (w_ & 0xFFFFu) * 16, dB_ = (w_ >> 16) * 16;                                                 \
    _Pragma("unroll") for (int i_ = 0; i_ < 4; ++i_) *(u32x4*)(smem_raw + dA_ + i_ * 4096) = fd##E[i_];              \
    _Pragma("unroll") for (int i_ = 0; i_ < 4; ++i_) *(u32x4*)(smem_raw + dB_ + i_ * 4096) = fd##E[4 + i_];          \
  }
    // one step: bA_/gA_/sA_ base, first byte offset and piece distance of pieces 0..3, bB_/gB_/sB_ of pieces 4..7;
    // dA_ / dB_ destination units of the two halves inside the slot
#define WQ_PROC(E, bA_, gA_, sA_, bB_, gB_, sB_, dAu_, dBu_)                                                         \
  {                                                                                                                  \
    if (L >= 3) __syncthreads();                                                                                     \
    /* piece by piece: the old content of a register goes to LDS, then the register is requested anew, so that the */ \
    /* LDS port and the vector-memory path of the CU work side by side instead of one after the other */             \
    const uint32_t w_ = fw##E;                                                                                       \
    const uint32_t oA_ = (w_ & 0xFFFFu) * 16, oB_ = (w_ >> 16) * 16;                                                 \
    const bool st_ = L >= 2;                                                                                         \
    _Pragma("unroll") for (int i_ = 0; i_ < 4; ++i_) {                                                               \
      if (st_) *(u32x4*)(smem_raw + oA_ + i_ * 4096) = fd##E[i_];                                                    \
      fd##E[i_] = *(const u32x4*)((bA_) + ((gA_) + i_ * (sA_)));                                                     \
    }                                                                                                                \
    _Pragma("unroll") for (int i_ = 0; i_ < 4; ++i_) {                                                               \
      if (st_) *(u32x4*)(smem_raw + oB_ + i_ * 4096) = fd##E[4 + i_];                                                \
      fd##E[4 + i_] = *(const u32x4*)((bB_) + ((gB_) + i_ * (sB_)));                                                 \
    }                                                                                                                \
    fw##E = ((dAu_) + (E) * (kWqSlot / 16)) | (((dBu_) + (E) * (kWqSlot / 16)) << 16);                               \
    ++L;                                                                                                             \
  }
    WqItem it;
    for (int rd = 0; rd < n_rounds; ++rd) {
      if (!wq_decode(it, rd, vid, G, n_items, NWIN)) continue;
      const uint32_t pl = (uint32_t)opaque(p);
      const char* const dH_b = (const char*)a.dH + (size_t)it.bh * S * DHHV * 2;
      const char* const V_b = (const char*)a.V + (size_t)it.bh * S * DHHV * 2;
      const char* const K_b = (const char*)a.K + (size_t)it.bh * S * DHQK * 2;
      const char* const Q_b = (const char*)a.Q + (size_t)it.bh * S * DHQK * 2;
      const size_t st_ofs = ((size_t)it.bh * NWIN + it.win) * (size_t)(DHHV / 32) * ND * 1024;
      const char* const C_b = (const char*)a.states + st_ofs;
      const char* const dC_b = (const char*)a.states2 + st_ofs;
      const uint32_t t0 = (uint32_t)it.win * 256;  // first position of the window
      // operand rows x 32 value columns: piece (row, unit) = (pl / 4 + 64 i, pl % 4), 64 bytes per row and slab
      const uint32_t xrow = pl >> 2, xun = pl & 3;
      const uint32_t xdu = xrow * 4 + (xun ^ (uint32_t)wq_f64((int)xrow));
      const uint32_t xg = (t0 + xrow) * (uint32_t)(DHHV * 2) + xun * 16;
      const uint32_t xstep = 64 * (uint32_t)DHHV * 2;
      // state fragments of 32 value columns: 16 KB contiguous in memory; lanes 32..63 of every fragment are stored 4
      // slots off so that the two lane halves a transposing read touches together fall on different LDS banks
      const uint32_t cdu = pl ^ (((pl >> 5) & 1) << 2);
      // 64 rows x 256 head-dim entries: piece (row, unit) = (pl / 32 + 8 i, pl % 32), 512 bytes per row
      const uint32_t zrow = pl >> 5, zun = pl & 31;
      const uint32_t zdu = zrow * 32 + (zun ^ (2 * (zrow & 3)));
      const uint32_t zg = (t0 + zrow) * (DHQK * 2) + zun * 16;
      // (every loop works on its own opaque copy of the offsets: addresses shared between two loops would otherwise be
      // kept, and spilled, across everything in between)
#define WQ_ROWS(bA_, bB_)                                                                                            \
  {                                                                                                                  \
    const uint32_t zz = (uint32_t)opaque((int)zg);                                                                   \
    for (int z = 0; z < 4; z += 2) {                                                                                 \
      WQ_PROC(0, bA_, zz + z * 32768, 4096, bB_, zz + z * 32768 + 16384, 4096, zdu, 1024 + zdu)                      \
      WQ_PROC(1, bA_, zz + (z + 1) * 32768, 4096, bB_, zz + (z + 1) * 32768 + 16384, 4096, zdu, 1024 + zdu)          \
    }                                                                                                                \
  }
      // ---- phase S: dH rows | V rows
      {
        const uint32_t xx = (uint32_t)opaque((int)xg);
        for (int w = 0; w < NV; w += 2) {
          WQ_PROC(0, dH_b, xx + w * 64, xstep, V_b, xx + w * 64, xstep, xdu, 1024 + xdu)
          WQ_PROC(1, dH_b, xx + (w + 1) * 64, xstep, V_b, xx + (w + 1) * 64, xstep, xdu, 1024 + xdu)
        }
      }
      // ---- phase Q: C fragments | dH rows, then the K rows (products) and the Q rows (row dots)
      {
        const uint32_t xx = (uint32_t)opaque((int)xg), cc = (uint32_t)opaque((int)(pl * 16));
        for (int w = 0; w < NV; w += 2) {
          WQ_PROC(0, C_b, (uint32_t)w * 16384 + cc, 4096, dH_b, xx + w * 64, xstep, cdu, 1024 + xdu)
          WQ_PROC(1, C_b, (uint32_t)(w + 1) * 16384 + cc, 4096, dH_b, xx + (w + 1) * 64, xstep, cdu, 1024 + xdu)
        }
      }
      WQ_ROWS(K_b, K_b)
      WQ_ROWS(Q_b, Q_b)
      // ---- phase K: dC fragments | V rows, then the Q rows (products) and the K rows (row dots)
      {
        const uint32_t xx = (uint32_t)opaque((int)xg), cc = (uint32_t)opaque((int)(pl * 16));
        for (int w = 0; w < NV; w += 2) {
          WQ_PROC(0, dC_b, (uint32_t)w * 16384 + cc, 4096, V_b, xx + w * 64, xstep, cdu, 1024 + xdu)
          WQ_PROC(1, dC_b, (uint32_t)(w + 1) * 16384 + cc, 4096, V_b, xx + (w + 1) * 64, xstep, cdu, 1024 + xdu)
        }
      }
      WQ_ROWS(Q_b, Q_b)
      WQ_ROWS(K_b, K_b)
#undef WQ_ROWS
    }
    // ---- drain: the last two slabs go to LDS, then the barriers of the consumers' last steps and of the final row dots
    if (L > 0) {
      if (L >= 3) __syncthreads();
      WQ_STORE(0)
      __syncthreads();
      WQ_STORE(1)
      __syncthreads();
      __syncthreads();
    }
#undef WQ_PROC
#undef WQ_STORE
  } else {
    // =========================================================================================== consumer waves
    const int wave = wave_all;
    const int tid = wave * 64 + lane;
    const int di = wave & 3, par = wave >> 2;  // head-dim rows 64 di .., position blocks 2 nb + par (nb = 0 .. 3)
    unsigned char* const stg = smem_raw + kWqStgOfs + wave * 2048;
    const uint64_t sblk = wq_score_blocks(wave);
    const int n_sblk = (int)((sblk >> 30) & 7);
    f32x16 acc[2][4];
    WqItem it, prev;
    prev = WqItem{0, 0};
    int pending = 0;       // row dots waiting in `red`: 1 dQ of `prev`, 2 dK of `prev`
    uint32_t slot = 0;     // ring slot of the next slab
    auto next_slab = [&]() {
      const unsigned char* s = smem_raw + slot * kWqSlot;
      slot ^= 1;
      return s;
    };
    // row dots of the last finished phase: the four 64-row blocks' partials meet in LDS, 256 threads add them up
    auto finish_rowdots = [&]() {
      if (pending && tid < 256) {
        const float dot = (red[tid] + red[256 + tid]) + (red[512 + tid] + red[768 + tid]);
        (pending == 2 ? a.rowdot2 : a.rowdot)[(size_t)prev.bh * Sp + (size_t)prev.win * 256 + tid] = dot;
      }
      pending = 0;
    };

    for (int rd = 0; rd < n_rounds; ++rd) {
      if (!wq_decode(it, rd, vid, G, n_items, NWIN)) continue;
      const int bh = it.bh, c0 = 2 * it.win;
      const size_t hofs = (size_t)bh * Sp, gofs = hofs + (size_t)c0 * kChunk;
      const float* graw = a.g.graw + (size_t)bh * NC;
      const float* mst = a.g.mstates + (size_t)bh * (NC + 1);
      const float g01 = graw[c0];   // decay over chunk c0: what separates a position of c1 from the keys of c0

      // ================================================================================= phase S: the score blocks
      {
        // gate vectors of the window, requested now, written to LDS after the first step
        float pu = 0.f, pw = 0.f, pr = 1.f;
        if (tid < 256) {
          pu = a.g.u[gofs + tid];
          pw = a.g.w[gofs + tid];
          if (a.use_nrow) pr = a.nrow[gofs + tid];
        }
        f32x16 sacc[5];
#pragma unroll
        for (int e = 0; e < 5; ++e)
#pragma unroll
          for (int i = 0; i < 16; ++i) sacc[e][i] = 0.f;
        for (int w = 0; w < NV; ++w) {
          __syncthreads();
          const unsigned char* const slab = next_slab();
          if (w == 0) {
            finish_rowdots();
            prev = it;
          }
          if (w == (NV > 2 ? 1 : 0)) {
            if (tid < 256) {
              uvec[tid] = pu;
              wvec[tid] = pw;
              lqr[tid] = __log2f(a.qk_scale * (a.use_nrow ? 1.f / (pr + a.eps) : 1.f));
            }
          }
          const int le = opaque(lane);
          const int r = le & 31, h = le >> 5;
#pragma unroll
          for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
            for (int e = 0; e < 5; ++e) {
              const int tb = (int)((sblk >> (6 * e)) & 7), jb = (int)((sblk >> (6 * e + 3)) & 7);
              const int trow = 32 * tb + r, jrow = 32 * jb + r;
              Frag A, B;
              B.u = *(const uint4*)(slab + trow * 64 + (((2 * ks + h) ^ wq_f64(trow)) * 16));
              A.u = *(const uint4*)(slab + 16384 + jrow * 64 + (((2 * ks + h) ^ wq_f64(jrow)) * 16));
              mfma32<F16>(sacc[e], A, B);   // rows: keys j, columns: positions t
            }
          }
        }
        // ---- gating: P[t][j] = scores * exp(u_t - w_j + G) / sqrt(DHQK) * rho_t, zero above the diagonal.  The
        // vectors were written after the first barrier of this phase and NV - 1 >= 1 barriers have passed since.
        {
          const int le = opaque(lane);
          const int r = le & 31, h = le >> 5;
#pragma unroll
          for (int e = 0; e < 5; ++e) {
            if (e < n_sblk) {
              const int tb = (int)((sblk >> (6 * e)) & 7), jb = (int)((sblk >> (6 * e + 3)) & 7);
              const float gg = (tb >= 4 && jb < 4) ? g01 : 0.f;
              const float un = uvec[32 * tb + r] + gg;
              const float lq = lqr[32 * tb + r];
              unsigned char* const pb = smem_raw + kWqPOfs + (tb * (tb + 1) / 2 + jb) * 2048 + r * 64;
              const int fr = wq_f64(r);
#pragma unroll
              for (int g4 = 0; g4 < 4; ++g4) {
                const int j0 = 8 * g4 + 4 * h;
                const float4 wj = *(const float4*)(wvec + 32 * jb + j0);
                const float wv[4] = {wj.x, wj.y, wj.z, wj.w};
                float pv[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                  const float e2 = __builtin_amdgcn_exp2f(__builtin_fmaf(un - wv[q], kWqLog2e, lq));
                  const bool keep = tb != jb || j0 + q <= r;
                  pv[q] = keep ? sacc[e][4 * g4 + q] * e2 : 0.f;
                }
                *(uint2*)(pb + ((g4 ^ fr) * 16) + 8 * h) = make_uint2(pack2<F16>(pv[0], pv[1]), pack2<F16>(pv[2], pv[3]));
              }
            }
          }
        }
      }

      // ============================================================================ phases Q (dQ) and K (dK)
      auto run_phase = [&](auto DKT) {
        constexpr bool dk = decltype(DKT)::value;
        // column scale of the inter-chunk part: requested now by one thread per position, parked in LDS after the first
        // step of the value pass, used after its last one (registers are what this kernel is short of)
        float csn = 0.f;
        if (tid < 256) {
          const size_t gi = gofs + tid;
          if (dk) {
            const float xs = __expf(graw[c0 + 1] + mst[c0 + 1] - mst[c0 + 2]);   // keys of c0 see dC through chunk c1
            csn = a.g.abar[gi] * (tid < 128 ? xs : 1.f);
          } else {
            const float xs = __expf(g01 + mst[c0] - mst[c0 + 1]);                // positions of c1 see C through chunk c0
            const float rh = a.use_nrow ? 1.f / (a.nrow[gi] + a.eps) : 1.f;
            csn = a.g.bbar[gi] * a.qk_scale * rh * (tid >= 128 ? xs : 1.f);
          }
        }
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
          for (int nb = 0; nb < 4; ++nb)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.f;

        // ---- Out^T += State Xn^T over the value columns, 32 at a time.  The stored fragments (made for a contraction
        // over the head dimension) are read with the transposing LDS read: lane i16 of a 16-lane block addresses
        // value column k0 + i16 / 4 and the 4 consecutive head-dim rows n0 + 4 (i16 % 4) .. + 3
        for (int w = 0; w < NV; ++w) {
          __syncthreads();
          const unsigned char* const Cf = next_slab();
          if (w == 0) finish_rowdots();
          // (one step after the request, so that its latency hides behind the first step; read after the last step of
          // this loop, at least one barrier later)
          if (w == (NV > 2 ? 1 : 0) && tid < 256) csv[tid] = csn;
          const unsigned char* const Xn = Cf + 16384;
          const int le = opaque(lane);
          const int r = le & 31, h = le >> 5;
          const int q16 = (le >> 4) & 1, i16 = le & 15;
          const int d_grp = i16 & 3;
          const int h_src = d_grp & 1, a_src = d_grp >> 1;
#pragma unroll
          for (int ks = 0; ks < 2; ++ks) {
            Frag A[2], B[4];
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) {
              const int row = 32 * (2 * nb + par) + r;
              B[nb].u = *(const uint4*)(Xn + row * 64 + (((2 * ks + h) ^ wq_f64(row)) * 16));
            }
            const int wrow = 16 * ks + 8 * h + (i16 >> 2);  // value column inside the 32-column slab (first read)
#pragma unroll
            for (int mb = 0; mb < 2; ++mb) {
              const int ds_l = (64 * di + 32 * mb + 16 * q16) / 16;
#pragma unroll
              for (int half = 0; half < 2; ++half) {
                const int wr = wrow + 4 * half;
                const int slot_l = (32 * h_src + wr) ^ (h_src << 2);
                A[mb].d[half] = lds_read_tr16(Cf + ((size_t)ds_l * 64 + slot_l) * 16 + 8 * a_src);
              }
            }
#pragma unroll
            for (int mb = 0; mb < 2; ++mb)
#pragma unroll
              for (int nb = 0; nb < 4; ++nb) mfma32<F16>(acc[mb][nb], A[mb], B[nb]);
          }
        }
        // column scale of the inter-chunk part (kept apart from the matrix instructions around it)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
          const float cs = csv[32 * (2 * nb + par) + (opaque(lane) & 31)];
#pragma unroll
          for (int mb = 0; mb < 2; ++mb) acc[mb][nb] *= cs;
        }
        __builtin_amdgcn_sched_barrier(0);

        // ---- Out^T += Z^T P'^T over the 256 positions of the window, 64 rows of Z per slab (Z = K for dQ with
        // P' = P: contraction over the keys j; Z = Q for dK with P' = P^T: contraction over the positions t)
        for (int z = 0; z < 4; ++z) {
          __syncthreads();
          const unsigned char* const Zs = next_slab();
          const int le = opaque(lane);
          const int r = le & 31, h = le >> 5;
          const int q16 = (le >> 4) & 1, i16 = le & 15;
          const int krow = 8 * h + (i16 >> 2);
          const int zun = 2 * q16 + ((i16 & 3) >> 1), zin = 8 * (i16 & 1);   // 16-byte unit and byte inside it
#pragma unroll
          for (int zh = 0; zh < 2; ++zh) {
            const int ob = 2 * z + zh;  // 32-position block of the contraction index
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
              Frag A[2];
#pragma unroll
              for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                  const int row = 32 * zh + 16 * kk + krow + 4 * half;
                  const int un = 8 * di + 4 * mb + zun;
                  A[mb].d[half] = lds_read_tr16(Zs + row * 512 + ((un ^ (2 * (row & 3))) * 16) + zin);
                }
#pragma unroll
              for (int nb = 0; nb < 4; ++nb) {
                const int nbk = 2 * nb + par;   // the wave's position block (dQ: t, dK: j)
                const bool live = dk ? ob >= nbk : ob <= nbk;
                // (the matrix instructions stay unconditional: accumulators that pass through a branch get copied;
                // a block above the diagonal contributes an operand of zeros instead)
                Frag B;
                B.u = make_uint4(0u, 0u, 0u, 0u);
                if (live) {
                  if (dk) {
                    // P^T: rows t of block (ob, nbk) are the contraction index -> transposing read
                    const unsigned char* const pb = smem_raw + kWqPOfs + (ob * (ob + 1) / 2 + nbk) * 2048;
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
                      const int row = 16 * kk + krow + 4 * half;
                      B.d[half] = lds_read_tr16(pb + row * 64 + ((zun ^ wq_f64(row)) * 16) + zin);
                    }
                  } else {
                    const unsigned char* const pb = smem_raw + kWqPOfs + (nbk * (nbk + 1) / 2 + ob) * 2048;
                    B.u = *(const uint4*)(pb + r * 64 + (((2 * kk + h) ^ wq_f64(r)) * 16));
                  }
                }
#pragma unroll
                for (int mb = 0; mb < 2; ++mb) mfma32<F16>(acc[mb][nb], A[mb], B);
              }
            }
          }
        }

        // ---- results, 64 positions per step: the x rows (q for dQ, k for dK) of those positions arrive as one more
        // slab; every wave owns one 32-position block of them.  Row dots sum_d x Out from the fp32 accumulators (they
        // feed a suffix sum over the whole sequence, where the rounding noise of 16-bit outputs would add up); then
        // the rounded values pass, 16 positions at a time, through the wave's private staging tile into row order and
        // leave as full 128-byte lines.
        char* const Ob = (char*)(dk ? a.Out2 : a.Out) + ((size_t)bh * S + (size_t)c0 * kChunk) * (DHQK * 2);
#pragma unroll
        for (int z = 0; z < 4; ++z) {
          __syncthreads();
          const unsigned char* const Xs = next_slab();
          const int le = opaque(lane);
          const int r = le & 31, h = le >> 5;
          {
            const int row = 32 * par + r;
            const unsigned char* const xrow = Xs + row * 512 + 8 * h;
            const int sw = 2 * (row & 3);
            float part = 0.f;
#pragma unroll
            for (int mb = 0; mb < 2; ++mb)
#pragma unroll
              for (int g4 = 0; g4 < 4; ++g4) {
                const uint2 xv = *(const uint2*)(xrow + (((8 * di + 4 * mb + g4) ^ sw) * 16));
                part += acc[mb][z][4 * g4 + 0] * lo2<F16>(xv.x);
                part += acc[mb][z][4 * g4 + 1] * hi2<F16>(xv.x);
                part += acc[mb][z][4 * g4 + 2] * lo2<F16>(xv.y);
                part += acc[mb][z][4 * g4 + 3] * hi2<F16>(xv.y);
              }
            part += __shfl_xor(part, 32);
            if (h == 0) red[di * 256 + 64 * z + row] = part;
          }
          const uint32_t lofs = (uint32_t)((le >> 3) * (DHQK * 2) + 128 * di + 16 * (le & 7));
#pragma unroll
          for (int q = 0; q < 2; ++q) {
            if ((r >> 4) == q) {
              const int row = r & 15;
#pragma unroll
              for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4)
                  *(uint2*)(stg + row * 128 + (((4 * mb + g4) ^ (row & 7)) * 16) + 8 * h) =
                      make_uint2(pack2<F16>(acc[mb][z][4 * g4 + 0], acc[mb][z][4 * g4 + 1]),
                                 pack2<F16>(acc[mb][z][4 * g4 + 2], acc[mb][z][4 * g4 + 3]));
            }
            __builtin_amdgcn_wave_barrier();
            const int row8 = le >> 3, un = le & 7;
            const u32x4 o0 = *(const u32x4*)(stg + row8 * 128 + ((un ^ row8) * 16));
            const u32x4 o1 = *(const u32x4*)(stg + (row8 + 8) * 128 + ((un ^ row8) * 16));
            __builtin_amdgcn_wave_barrier();
            const uint32_t n0 = (uint32_t)(64 * z + 32 * par + 16 * q);
            __builtin_nontemporal_store(o0, (u32x4*)(Ob + (lofs + n0 * (DHQK * 2))));
            __builtin_nontemporal_store(o1, (u32x4*)(Ob + (lofs + (n0 + 8) * (DHQK * 2))));
          }
        }
        pending = dk ? 2 : 1;
      };
      run_phase(std::false_type{});
      run_phase(std::true_type{});
    }
    if (pending) {   // (a workgroup without a window passes no barrier at all, like its producers)
      __syncthreads();
      finish_rowdots();
    }
  }
}

bool window_qk_supported(const ParQkArgs& a) {
  return a.stride == 2 && a.DHQK == 256 && a.DHHV % 64 == 0 && a.S % (2 * kChunk) == 0;
}

namespace {
int wq_device_cu_count() {
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
const char* launch_window_qk_t(const ParQkArgs& a, int BH, hipStream_t stream) {
  const long long n_items = (long long)BH * (a.NC / 2);
  if (n_items >= (1ll << 31)) return "window_qk: too many work items";
  if ((size_t)a.S * (size_t)(a.DHHV > a.DHQK ? a.DHHV : a.DHQK) * 2 >= ((size_t)1 << 32))
    return "window_qk: one (batch, head) slab of an input exceeds 4 GiB";
  const int cus = wq_device_cu_count();
  if (cus <= 0) return "window_qk: cannot read the number of compute units";
  int G = (int)(n_items < cus ? n_items : cus);
  if (G >= 8) G -= G % 8;
  const int n_rounds = (int)((n_items + G - 1) / G);
  if (hipFuncSetAttribute((const void*)window_qk_kernel<F16>, hipFuncAttributeMaxDynamicSharedMemorySize, kWqSmem) != hipSuccess)
    return "window_qk: cannot raise the dynamic LDS limit";
  hipLaunchKernelGGL((window_qk_kernel<F16>), dim3(G), dim3(768), kWqSmem, stream, a, (int)n_items, n_rounds);
  return nullptr;
}
}  // namespace

const char* launch_window_qk(const ParQkArgs& a, int BH, hipStream_t stream) {
  if (!window_qk_supported(a)) return "window_qk: unsupported shape (needs state stride 2, DHQK = 256, DHHV % 64 == 0, S % 256 == 0)";
  if (a.states2 == nullptr || a.Out2 == nullptr || a.rowdot2 == nullptr) return "window_qk: the dK operands are missing";
  return a.f16 ? launch_window_qk_t<true>(a, BH, stream) : launch_window_qk_t<false>(a, BH, stream);
}

}  // namespace mlstm
