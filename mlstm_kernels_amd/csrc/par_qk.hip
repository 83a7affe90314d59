// Chunk-parallel backward kernels whose output tile spans the query/key head dimension: dQ and dK.
//
// (mlstm_kernels/torch/chunkwise/native/bw.py:153-198 in the reference), per chunk, rho_t = 1/(nrow_t + eps):
//   dS[t][j] = exp(u_t - w_j)/sqrt(DHQK) * rho_t * (dH_t . v_j)                                (j <= t)
//   dQ[t][:] = sum_j dS[t][j] k_j  +  bbar_t/sqrt(DHQK) * rho_t * C_prev dH_t
//   dK[j][:] = sum_t dS[t][j] q_t  +  abar_j * dC_next v_j
//
// Chunk states are kept only every `stride`-th chunk.  A chunk whose own boundary state was not kept uses the nearest
// kept one (dQ: at or before the chunk, dK: at or after it) with the decay over the chunks in between folded into the
// column scale, and adds those chunks as further score blocks without a causal mask,
//   dS'[t][j] = exp(u_t - w_j + G)/sqrt(DHQK) * rho_t * (dH_t . v_j),   G = sum of logsig(f) over the chunks from the
// key's chunk up to (not including) the query's chunk -- the same algebra as in the H / dV kernels.
//
// Both gradients are one GEMM chain on the transposed output tile  Out^T[d][n]  (head dimension x chunk positions):
//   Out^T = ( State[d][w] . Xn^T[w][n] ) * colscale[n]  +  sum over source chunks  Z^T[d][o] . P[o][n]
// with  n = t, o = j, Xn = dH, Xo = V,  Z = K, State = C    (dQ)
//       n = j, o = t, Xn = V,  Xo = dH, Z = Q, State = dC   (dK)
// and the score block  P[o][n] = gate * (Xo Xn^T)  contracted over the DHHV value columns.  For the chunk's own block
// one pass over DHHV in slabs of 32 columns feeds BOTH the inter-chunk product and the scores from the same Xn slab;
// every further source chunk costs one more pass over DHHV for its scores alone.  The state fragments (stored for a
// contraction over the head dimension) are copied to LDS unchanged and re-read with the transposing LDS read, which
// hands out operands for a contraction over value columns.  Row sums  sum_d x[n][d] * Out[n][d]  (x = q for dQ, k for
// dK) are emitted for the gate gradients, one slot per head-dimension tile (summed in a fixed order by the gate-gradient
// kernel, so the gate gradients are reproducible run to run).
//
// A workgroup owns MT head-dim rows x 64 positions (half a chunk); two slabs are in flight from global memory into
// registers while a third is being multiplied, and the footprint (54 KB of LDS) lets two workgroups share a CU so
// that one computes while the other waits for memory.  dQ and dK run as ONE launch (par_qk_pair_kernel).
#include "common.h"
#include "kernels.h"

namespace mlstm {

template <int MT, bool IS_DQ, bool F16>
__device__ __forceinline__ void par_qk_body(const ParQkArgs& a, const BlockId blk, const int n_bh) {
  constexpr int NWAVE = MT / 64;    // each wave owns 64 head-dim rows = 2 MFMA row blocks
  constexpr int NTH = 64 * NWAVE;
  constexpr int PS = 128 + 8;       // P stored as Ps[n][o]
  constexpr int XS = 64 + 8;        // row stride of the Xn / Xo slabs (64 value columns: two state slabs)
  constexpr int ZS = MT + 32;       // pass-2 slab row stride (rows 64 bytes apart in the banks)
  constexpr int OS = MT + 8;        // output staging row stride
  constexpr int NDT = MT / 16;      // 16-row state fragments per 32 value columns inside the tile
  constexpr int CF = NDT * 64 * 8;  // elements of the staged state fragments per 32-column slab
  const int DHQK = a.DHQK, DHHV = a.DHHV, S = a.S, NC = a.NC;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  // stage region: [state frags | Xn slab | Xo slab], later pass-2 slabs, later the output staging tile
  constexpr int stage_elems_a = CF + 64 * XS + 128 * XS;
  constexpr int stage_elems_b = 64 * OS;
  constexpr int stage_elems_c = 64 * ZS;
  constexpr int stage_ab = stage_elems_a > stage_elems_b ? stage_elems_a : stage_elems_b;
  constexpr int stage_elems = stage_ab > stage_elems_c ? stage_ab : stage_elems_c;
  uint16_t* Cf = (uint16_t*)smem_raw;
  uint16_t* Xn = Cf + CF;
  uint16_t* Xo = Xn + 64 * XS;
  uint16_t* Ps = Cf + stage_elems;
  float* nvec = (float*)(Ps + 64 * PS);  // [64] gate vector of this workgroup's positions: u_t (dQ) / w_j (dK)
  float* nrho = nvec + 64;             // [64] dQ: rho_t of this workgroup's positions
  float* ovec = nrho + 64;             // [128] gate vector of the source chunk: w_j (dQ) / u_t (dK)
  float* orho = ovec + 128;            // [128] dK: rho_t of the source chunk
  float* cs = orho + 128;              // [64] column scale of this workgroup's positions
  float* red = cs + 64;                // [NWAVE][64] row-dot partials

  // the wave index is made scalar so that branches on it are scalar branches (accumulators stay in place)
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, h = lane >> 5;
  const int bh = blk.z, c = blk.y;
  const int nh = blk.x & 1;
  const int d_idx = blk.x >> 1;
  const int d_tile = d_idx * MT;
  const size_t Sp = (size_t)NC * kChunk;
  const size_t hofs = bh * Sp;
  const size_t gofs = hofs + (size_t)c * kChunk;
  const int t_base = c * kChunk;
  const int n0 = 64 * nh;
  const int stride = a.stride;
  const int slot = c / stride;
  // source chunks of the score blocks: dQ c0 .. c, dK c .. c1; the own chunk is handled first, together with the state
  const int sc_lo = IS_DQ ? slot * stride : c;
  const int sc_hi = IS_DQ ? c : min(slot * stride + stride - 1, NC - 1);
  // live 32-row blocks of the other position index in the own chunk: dQ o = j <= t, dK o = t >= j
  const int ob_lo = IS_DQ ? 0 : 2 * nh, ob_hi = IS_DQ ? 2 * (nh + 1) : 4;
  const uint16_t* Xn_g = (IS_DQ ? a.dH : a.V) + (size_t)bh * S * DHHV;
  const uint16_t* Xo_g = (IS_DQ ? a.V : a.dH) + (size_t)bh * S * DHHV;
  const uint16_t* Z_g = (IS_DQ ? a.K : a.Q) + (size_t)bh * S * DHQK + d_tile;
  const float* graw = a.g.graw + (size_t)bh * NC;
  const float* mst = a.g.mstates + (size_t)bh * (NC + 1);

  for (int idx = tid; idx < 128; idx += NTH) {
    ovec[idx] = (IS_DQ ? a.g.w : a.g.u)[gofs + idx];
    if (!IS_DQ) orho[idx] = a.use_nrow ? 1.f / (a.nrow[gofs + idx] + a.eps) : 1.f;
  }
  if (tid < 64) {
    // weight of the kept boundary state for this chunk (1 when the boundary is the chunk's own)
    float gsum = 0.f, xs;
    if (IS_DQ) {
      for (int x = sc_lo; x < c; ++x) gsum += graw[x];
      xs = sc_lo < c ? __expf(gsum + mst[sc_lo] - mst[c]) : 1.f;
    } else {
      for (int x = c + 1; x <= sc_hi; ++x) gsum += graw[x];
      xs = sc_hi > c ? __expf(gsum + mst[c + 1] - mst[sc_hi + 1]) : 1.f;
    }
    const float rh = a.use_nrow ? 1.f / (a.nrow[gofs + n0 + tid] + a.eps) : 1.f;
    cs[tid] = (IS_DQ ? a.g.bbar[gofs + n0 + tid] * a.qk_scale * rh : a.g.abar[gofs + n0 + tid]) * xs;
    nvec[tid] = (IS_DQ ? a.g.u : a.g.w)[gofs + n0 + tid];
    nrho[tid] = IS_DQ ? rh : 1.f;
  }

  constexpr int OBW = (4 + NWAVE - 1) / NWAVE;  // score blocks per wave (at most)
  f32x16 acc[2][2], sacc[OBW][2];
#pragma unroll
  for (int mb = 0; mb < 2; ++mb)
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.f;
#pragma unroll
  for (int k = 0; k < OBW; ++k)
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) sacc[k][nb][i] = 0.f;
  const int m_wave = wave * 64;
  const int q16 = (lane >> 4) & 1, i16 = lane & 15;
  const int nslab = DHHV / 32;  // even: DHHV is a multiple of 64

  // The Xn / Xo rows are fetched 64 columns at a time (one fetch serves two state slabs): 128 contiguous bytes per row
  // and load instruction instead of 64.
  constexpr int NV = 64 * 8 / NTH;        // Xn vectors per thread per pair of slabs
  constexpr int OV = 128 * 8 / NTH;       // Xo vectors per thread per pair of slabs
  uint4 nreg[NV], oreg[OV];
  // (macros, not lambdas: with the arrays captured by reference the compiler kept them in scratch memory)
  // source chunk sc_, live blocks lo_ .. hi_ - 1 of it, columns 64 * pair_ .. + 63
#define MLSTM_LOAD_X(sc_, lo_, hi_, pair_)                                                                           \
  {                                                                                                                  \
    _Pragma("unroll") for (int v = 0; v < NV; ++v) {                                                                 \
      const int idx = tid + v * NTH;                                                                                 \
      const int t = t_base + n0 + (idx >> 3);                                                                        \
      nreg[v] = t < S ? *(const uint4*)(Xn_g + (size_t)t * DHHV + (pair_) * 64 + (idx & 7) * 8) : make_uint4(0, 0, 0, 0); \
    }                                                                                                                \
    _Pragma("unroll") for (int v = 0; v < OV; ++v) {                                                                 \
      const int idx = tid + v * NTH;                                                                                 \
      const int j = idx >> 3;                                                                                        \
      const int t = (sc_) * kChunk + j;                                                                              \
      const bool live = j >= 32 * (lo_) && j < 32 * (hi_) && t < S;                                                  \
      oreg[v] = live ? *(const uint4*)(Xo_g + (size_t)t * DHHV + (pair_) * 64 + (idx & 7) * 8) : make_uint4(0, 0, 0, 0); \
    }                                                                                                                \
  }
#define MLSTM_STORE_X                                                                                                \
  {                                                                                                                  \
    _Pragma("unroll") for (int v = 0; v < NV; ++v) {                                                                 \
      const int idx = tid + v * NTH;                                                                                 \
      *(uint4*)(Xn + (idx >> 3) * XS + (idx & 7) * 8) = nreg[v];                                                     \
    }                                                                                                                \
    _Pragma("unroll") for (int v = 0; v < OV; ++v) {                                                                 \
      const int idx = tid + v * NTH;                                                                                 \
      *(uint4*)(Xo + (idx >> 3) * XS + (idx & 7) * 8) = oreg[v];                                                     \
    }                                                                                                                \
  }
  // score part of one staged 32-column slab: A = Xo rows of the blocks dealt to this wave, B = Xn rows
#define MLSTM_SCORE_SLAB(sub_, lo_)                                                                                  \
  _Pragma("unroll") for (int ks = 0; ks < 2; ++ks) {                                                                 \
    Frag B[2];                                                                                                       \
    _Pragma("unroll") for (int nb = 0; nb < 2; ++nb)                                                                 \
      B[nb].u = *(const uint4*)(Xn + (32 * nb + r) * XS + 32 * (sub_) + 16 * ks + 8 * h);                            \
    _Pragma("unroll") for (int k = 0; k < OBW; ++k) {                                                                \
      const int ob = (lo_) + wave + k * NWAVE;                                                                       \
      const int obc = ob < 4 ? ob : 3;                                                                               \
      Frag A;                                                                                                        \
      A.u = *(const uint4*)(Xo + (32 * obc + r) * XS + 32 * (sub_) + 16 * ks + 8 * h);                               \
      _Pragma("unroll") for (int nb = 0; nb < 2; ++nb) mfma32<F16>(sacc[k][nb], A, B[nb]);                                \
    }                                                                                                                \
  }

  // ---- pass 1 over the value columns: inter-chunk product and the scores of the own chunk
  {
    const size_t ND = DHQK / 16, NW = DHHV / 32;
    const size_t NCS = (size_t)(NC + stride - 1) / stride;
    const u32x4* st = (const u32x4*)a.states + ((size_t)bh * NCS + slot) * NW * ND * 64;
    constexpr int CV = NDT * 64 / NTH;      // state-fragment vectors per thread per slab
    // The state fragments come in slabs of 32 value columns, two slabs in flight in registers.
    u32x4 cregA[CV], cregB[CV];
#define MLSTM_LOAD_C(slab_, creg)                                                                                    \
  {                                                                                                                  \
    _Pragma("unroll") for (int v = 0; v < CV; ++v)                                                                   \
        creg[v] = st[((size_t)(slab_) * ND + d_tile / 16) * 64 + tid + v * NTH];                                     \
  }
    // lanes 32..63 of every state fragment are stored 4 slots off so that the two lane halves a transposing read
    // touches together fall on different LDS banks
#define MLSTM_STORE_C(creg)                                                                                          \
  {                                                                                                                  \
    _Pragma("unroll") for (int v = 0; v < CV; ++v) {                                                                 \
      const int idx = tid + v * NTH;                                                                                 \
      ((u32x4*)Cf)[idx ^ (((idx >> 5) & 1) << 2)] = creg[v];                                                         \
    }                                                                                                                \
  }
    // transposing read of the staged fragments: lane i16 of a 16-lane block addresses value column
    // k0 + i16/4 and the 4 consecutive head-dim rows n0 + 4*(i16%4) .. +3
    const int d_grp = i16 & 3;
    const int h_src = d_grp & 1, a_src = d_grp >> 1;
    auto multiply_slab = [&](const int sub) {  // sub = which half of the staged Xn / Xo columns
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        Frag B[2];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
          B[nb].u = *(const uint4*)(Xn + (32 * nb + r) * XS + 32 * sub + 16 * ks + 8 * h);
        // inter-chunk product: A = State[d][w]
        {
          Frag A[2];
          const int wrow = 16 * ks + 8 * h + (i16 >> 2);  // value column inside the slab (first read)
#pragma unroll
          for (int mb = 0; mb < 2; ++mb) {
            const int ds_l = (m_wave + 32 * mb + 16 * q16) / 16;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
              const int wr = wrow + 4 * half;
              const int slot_l = (32 * h_src + wr) ^ (h_src << 2);
              const unsigned char* p = (const unsigned char*)Cf + ((size_t)ds_l * 64 + slot_l) * 16 + 8 * a_src;
              A[mb].d[half] = lds_read_tr16(p);
            }
          }
#pragma unroll
          for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) mfma32<F16>(acc[mb][nb], A[mb], B[nb]);
        }
        // score block: A = Xo rows of the blocks dealt to this wave.  Unconditional on purpose: a wave whose block lies
        // above the diagonal multiplies zero rows (its result is dropped at the gating step); a branch here would make
        // the compiler shuttle the score accumulators between the two register files on every iteration
#pragma unroll
        for (int k = 0; k < OBW; ++k) {
          const int ob = ob_lo + wave + k * NWAVE;
          const int obc = ob < 4 ? ob : 3;
          Frag A;
          A.u = *(const uint4*)(Xo + (32 * obc + r) * XS + 32 * sub + 16 * ks + 8 * h);
#pragma unroll
          for (int nb = 0; nb < 2; ++nb) mfma32<F16>(sacc[k][nb], A, B[nb]);
        }
      }
    };
    // two state slabs and one Xn / Xo pair are in flight in registers while a slab is multiplied: one memory round
    // trip spans two slab periods.  The prefetches are unconditional (the last iterations re-fetch the last slab): a
    // conditional prefetch makes the compiler keep the prefetch registers in scratch memory across the loop back-edge.
    MLSTM_LOAD_C(0, cregA)
    MLSTM_LOAD_X(c, ob_lo, ob_hi, 0)
    MLSTM_LOAD_C(1, cregB)
    for (int slab = 0; slab < nslab; slab += 2) {
      __syncthreads();
      MLSTM_STORE_C(cregA)
      MLSTM_STORE_X
      __syncthreads();
      MLSTM_LOAD_C(slab + 2 < nslab ? slab + 2 : nslab - 1, cregA)
      MLSTM_LOAD_X(c, ob_lo, ob_hi, slab + 2 < nslab ? slab / 2 + 1 : slab / 2)
      multiply_slab(0);
      __syncthreads();
      MLSTM_STORE_C(cregB)
      __syncthreads();
      MLSTM_LOAD_C(slab + 3 < nslab ? slab + 3 : nslab - 1, cregB)
      multiply_slab(1);
    }
#undef MLSTM_STORE_C
#undef MLSTM_LOAD_C
  }
  // column scale of the inter-chunk part
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const float sc = cs[32 * nb + r];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) acc[mb][nb] *= sc;
  }

  constexpr int ZV = 64 * (MT / 8) / NTH;
  uint4 zreg[ZV];
  auto load_zslab = [&](int sc, int ob) {  // 64 positions of source chunk sc, from block ob on
#pragma unroll
    for (int v = 0; v < ZV; ++v) {
      const int idx = tid + v * NTH;
      const int j = idx / (MT / 8), cv = idx % (MT / 8);
      const int t = sc * kChunk + 32 * ob + j;
      zreg[v] = t < S ? *(const uint4*)(Z_g + (size_t)t * DHQK + cv * 8) : make_uint4(0, 0, 0, 0);
    }
  };
  // gate the score block: P[o][n] = sacc * exp(u_t - w_j + G)/sqrt(DHQK) * rho_t (own chunk: for j <= t); store as
  // Ps[n][o].  lo_ .. hi_ - 1 are the live blocks of the source chunk, gs_ the decay G between the two chunks.
#define MLSTM_GATE_SCORES(lo_, hi_, own_, gs_)                                                                       \
  _Pragma("unroll") for (int k = 0; k < OBW; ++k) {                                                                  \
    const int ob = (lo_) + wave + k * NWAVE;                                                                         \
    if (ob < (hi_)) {                                                                                                \
      _Pragma("unroll") for (int nb = 0; nb < 2; ++nb) {                                                             \
        const int nl = 32 * nb + r;                                                                                  \
        const int n = n0 + nl;                                                                                       \
        const float xn = nvec[nl] + (IS_DQ ? (gs_) : -(gs_));                                                        \
        const float rn = nrho[nl];                                                                                   \
        _Pragma("unroll") for (int g4 = 0; g4 < 4; ++g4) {                                                           \
          const int o0 = 32 * ob + 8 * g4 + 4 * h;                                                                   \
          const float4 xo = *(const float4*)(ovec + o0);                                                             \
          const float xov[4] = {xo.x, xo.y, xo.z, xo.w};                                                             \
          float ro[4] = {1.f, 1.f, 1.f, 1.f};                                                                        \
          if (!IS_DQ) {                                                                                              \
            const float4 rr = *(const float4*)(orho + o0);                                                           \
            ro[0] = rr.x; ro[1] = rr.y; ro[2] = rr.z; ro[3] = rr.w;                                                  \
          }                                                                                                          \
          float pv[4];                                                                                               \
          _Pragma("unroll") for (int e = 0; e < 4; ++e) {                                                            \
            const float ex = IS_DQ ? (xn - xov[e]) : (xov[e] - xn);                                                  \
            const bool keep = !(own_) || (IS_DQ ? (o0 + e <= n) : (n <= o0 + e));                                    \
            const float val = sacc[k][nb][4 * g4 + e] * a.qk_scale * __expf(ex) * rn * ro[e];                        \
            pv[e] = keep ? val : 0.f;                                                                                \
          }                                                                                                          \
          *(uint2*)(Ps + nl * PS + o0) = make_uint2(pack2<F16>(pv[0], pv[1]), pack2<F16>(pv[2], pv[3]));           \
        }                                                                                                            \
      }                                                                                                              \
    }                                                                                                                \
  }
  // pass 2 over the live positions o of source chunk sc_: Out^T += Z^T P, 64 positions per slab (the live range is
  // always an even number of blocks); the first slab is already in zreg
#define MLSTM_PASS2(sc_, lo_, hi_)                                                                                   \
  {                                                                                                                  \
    uint16_t* Zs = Cf;                                                                                               \
    const int krow = 8 * h + (i16 >> 2), ncol = 16 * q16 + 4 * (i16 & 3);                                            \
    for (int ob = (lo_); ob < (hi_); ob += 2) {                                                                      \
      __syncthreads(); /* P written and the pass-1 slabs (or the previous pass-2 slab) consumed */                  \
      _Pragma("unroll") for (int v = 0; v < ZV; ++v) {                                                               \
        const int idx = tid + v * NTH;                                                                               \
        *(uint4*)(Zs + (idx / (MT / 8)) * ZS + (idx % (MT / 8)) * 8) = zreg[v];                                      \
      }                                                                                                              \
      __syncthreads();                                                                                               \
      if (ob + 2 < (hi_)) load_zslab((sc_), ob + 2);                                                                 \
      _Pragma("unroll") for (int jl = 0; jl < 4; ++jl) {                                                             \
        Frag A[2], B[2];                                                                                             \
        _Pragma("unroll") for (int mb = 0; mb < 2; ++mb) {                                                           \
          const uint16_t* p = Zs + (16 * jl + krow) * ZS + (m_wave + 32 * mb + ncol);                                \
          A[mb].d[0] = lds_read_tr16(p);                                                                             \
          A[mb].d[1] = lds_read_tr16(p + 4 * ZS);                                                                    \
        }                                                                                                            \
        _Pragma("unroll") for (int nb = 0; nb < 2; ++nb)                                                             \
          B[nb].u = *(const uint4*)(Ps + (32 * nb + r) * PS + 32 * ob + 16 * jl + 8 * h);                            \
        _Pragma("unroll") for (int mb = 0; mb < 2; ++mb)                                                             \
          _Pragma("unroll") for (int nb = 0; nb < 2; ++nb) mfma32<F16>(acc[mb][nb], A[mb], B[nb]);                        \
      }                                                                                                              \
    }                                                                                                                \
  }
  // the x rows of the row dots (q for dQ, k for dK) are fetched before the last pass 2 and parked in registers: their
  // memory round trip overlaps that pass instead of standing alone in the epilogue
  constexpr int XV = 64 * (MT / 8) / NTH;
  uint4 xreg[XV];
#define MLSTM_LOAD_XROWS                                                                                             \
  {                                                                                                                  \
    const uint16_t* Rg = (IS_DQ ? a.Q : a.K) + (size_t)bh * S * DHQK + d_tile;                                       \
    _Pragma("unroll") for (int v = 0; v < XV; ++v) {                                                                 \
      const int idx = tid + v * NTH;                                                                                 \
      const int j = idx / (MT / 8), cv = idx % (MT / 8);                                                             \
      const int t = t_base + n0 + j;                                                                                 \
      xreg[v] = t < S ? *(const uint4*)(Rg + (size_t)t * DHQK + cv * 8) : make_uint4(0, 0, 0, 0);                    \
    }                                                                                                                \
  }

  // ---- own chunk: first pass-2 slab into registers while the scores are gated
  load_zslab(c, ob_lo);
  const bool has_cross = sc_lo < sc_hi;
  if (!has_cross) MLSTM_LOAD_XROWS
  MLSTM_GATE_SCORES(ob_lo, ob_hi, true, 0.f)
  MLSTM_PASS2(c, ob_lo, ob_hi)

  // ---- further source chunks: one pass over the value columns for the scores, then pass 2 over all 128 positions
  for (int sc = sc_lo; sc <= sc_hi; ++sc) {
    if (sc == c) continue;
    float gs = 0.f;
    for (int x = (IS_DQ ? sc : c); x < (IS_DQ ? c : sc); ++x) gs += graw[x];
    constexpr int OVN = NTH >= 128 ? 1 : 128 / NTH;  // gate-vector entries per thread (a workgroup may be one wave)
    float ov[OVN], orh[OVN];
#pragma unroll
    for (int e = 0; e < OVN; ++e) {
      const int idx = tid + e * NTH;
      ov[e] = 0.f;
      orh[e] = 1.f;
      if (idx < 128) {
        ov[e] = (IS_DQ ? a.g.w : a.g.u)[hofs + (size_t)sc * kChunk + idx];
        if (!IS_DQ && a.use_nrow) orh[e] = a.nrow[hofs + (size_t)sc * kChunk + idx];
      }
    }
#pragma unroll
    for (int k = 0; k < OBW; ++k)
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int i = 0; i < 16; ++i) sacc[k][nb][i] = 0.f;
    MLSTM_LOAD_X(sc, 0, 4, 0)
    for (int pair = 0; pair < nslab / 2; ++pair) {
      __syncthreads();  // previous pair (or the previous pass 2) fully consumed
      MLSTM_STORE_X
      if (pair == 0) {
#pragma unroll
        for (int e = 0; e < OVN; ++e) {
          const int idx = tid + e * NTH;
          if (idx < 128) {
            ovec[idx] = ov[e];
            if (!IS_DQ) orho[idx] = a.use_nrow ? 1.f / (orh[e] + a.eps) : 1.f;
          }
        }
      }
      __syncthreads();
      MLSTM_LOAD_X(sc, 0, 4, pair + 1 < nslab / 2 ? pair + 1 : pair)
      MLSTM_SCORE_SLAB(0, 0)
      MLSTM_SCORE_SLAB(1, 0)
    }
    load_zslab(sc, 0);
    const bool last = IS_DQ ? (sc == c - 1) : (sc == sc_hi);
    if (last) MLSTM_LOAD_XROWS
    MLSTM_GATE_SCORES(0, 4, false, gs)
    MLSTM_PASS2(sc, 0, 4)
  }
#undef MLSTM_LOAD_X
#undef MLSTM_STORE_X
#undef MLSTM_SCORE_SLAB
#undef MLSTM_GATE_SCORES
#undef MLSTM_PASS2
#undef MLSTM_LOAD_XROWS
  __syncthreads();

  // ---- epilogue part 1: row dots  sum_d x[n][d] * Out[n][d]  from the fp32 accumulators (x = q for dQ, k for dK).
  // They feed a suffix sum over the whole sequence (dF), where the rounding noise of bf16 outputs would add up
  // like a random walk; the matching x rows are staged in LDS so every lane can read its own row.
  uint16_t* Os = Cf;
#pragma unroll
  for (int v = 0; v < XV; ++v) {
    const int idx = tid + v * NTH;
    *(uint4*)(Os + (idx / (MT / 8)) * OS + (idx % (MT / 8)) * 8) = xreg[v];
  }
  __syncthreads();
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int nl = 32 * nb + r;
    float part = 0.f;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int d0 = m_wave + 32 * mb + 8 * g4 + 4 * h;
        const uint2 xv = *(const uint2*)(Os + nl * OS + d0);
        part += acc[mb][nb][4 * g4 + 0] * lo2<F16>(xv.x);
        part += acc[mb][nb][4 * g4 + 1] * hi2<F16>(xv.x);
        part += acc[mb][nb][4 * g4 + 2] * lo2<F16>(xv.y);
        part += acc[mb][nb][4 * g4 + 3] * hi2<F16>(xv.y);
      }
    part += __shfl_xor(part, 32);
    if (h == 0) red[wave * 64 + nl] = part;
  }
  __syncthreads();
  if (tid < 64) {
    float dot = 0.f;
#pragma unroll
    for (int w = 0; w < NWAVE; ++w) dot += red[w * 64 + tid];
    // one slot per head-dimension tile: [tile][batch * head][position]
    a.rowdot[((size_t)d_idx * n_bh) * Sp + gofs + n0 + tid] = dot;
  }

  // ---- epilogue part 2: round, transpose through LDS, coalesced store
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int nl = 32 * nb + r;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int d0 = m_wave + 32 * mb + 8 * g4 + 4 * h;
        *(uint2*)(Os + nl * OS + d0) = make_uint2(pack2<F16>(acc[mb][nb][4 * g4 + 0], acc[mb][nb][4 * g4 + 1]),
                                                  pack2<F16>(acc[mb][nb][4 * g4 + 2], acc[mb][nb][4 * g4 + 3]));
      }
  }
  __syncthreads();
  {
    uint16_t* Og = a.Out + (size_t)bh * S * DHQK + d_tile;
    constexpr int vec_per_row = MT / 8;
    for (int idx = tid; idx < 64 * vec_per_row; idx += NTH) {
      const int j = idx / vec_per_row, cv = idx % vec_per_row;
      const int t = t_base + n0 + j;
      // non-temporal: nobody in this launch reads the output, it should not evict shared operands from the L2
      if (t < S) __builtin_nontemporal_store(*(const u32x4*)(Os + j * OS + cv * 8), (u32x4*)(Og + (size_t)t * DHQK + cv * 8));
    }
  }
}

#define PAR_QK_WPE(MT_) ((MT_) == 256 ? 2 : 1)
// dQ and dK of every chunk in ONE launch: the workgroups of a chunk (both gradients, both position halves, all
// head-dimension tiles) are neighbours in launch order and run on the same XCD at about the same time, so the Q, K, V
// and dH rows they all stream are fetched from HBM once and served to the others from the caches.
template <int MT, bool F16>
__global__ __launch_bounds__(MT) __attribute__((amdgpu_waves_per_eu(PAR_QK_WPE(MT), PAR_QK_WPE(MT)))) void par_qk_pair_kernel(ParQkArgs a) {
  BlockId blk = xcd_block_id();
  const int per = 2 * (a.DHQK / MT);
  const int n_bh = (int)gridDim.z;
  if (blk.x < per) {
    par_qk_body<MT, true, F16>(a, blk, n_bh);
  } else {
    blk.x -= per;
    a.states = a.states2;
    a.Out = a.Out2;
    a.rowdot = a.rowdot2;
    par_qk_body<MT, false, F16>(a, blk, n_bh);
  }
}

template <int MT, bool F16>
static const char* launch_par_qk_pair_f(const ParQkArgs& a, int BH, hipStream_t stream) {
  constexpr int CF = (MT / 16) * 64 * 8;
  constexpr int sa = CF + 64 * 72 + 128 * 72, sb = 64 * (MT + 8), sc = 64 * (MT + 32);
  constexpr int sab = sa > sb ? sa : sb;
  constexpr int stage = sab > sc ? sab : sc;
  const size_t smem = (size_t)(stage + 64 * 136) * 2 + (size_t)(64 * 2 + 128 * 2 + 64 + (MT / 64) * 64) * 4;
  if (hipFuncSetAttribute((const void*)par_qk_pair_kernel<MT, F16>, hipFuncAttributeMaxDynamicSharedMemorySize,
                          (int)smem) != hipSuccess)
    return "par_qk: cannot raise the dynamic LDS limit";
  dim3 grid(4 * (a.DHQK / MT), a.NC, BH);
  hipLaunchKernelGGL((par_qk_pair_kernel<MT, F16>), grid, dim3(MT), smem, stream, a);
  return nullptr;
}

template <int MT>
static const char* launch_par_qk_pair_t(const ParQkArgs& a, int BH, hipStream_t stream) {
  return a.f16 ? launch_par_qk_pair_f<MT, true>(a, BH, stream) : launch_par_qk_pair_f<MT, false>(a, BH, stream);
}

int par_qk_head_tile(int DHQK) { return DHQK % 256 == 0 ? 256 : (DHQK % 128 == 0 ? 128 : 64); }

const char* launch_par_qk_pair(const ParQkArgs& a, int BH, hipStream_t stream) {
  if (a.DHQK % 64 != 0 || a.DHHV % 64 != 0) return "par_qk: DHQK and DHHV must be multiples of 64";
  if (a.states2 == nullptr || a.Out2 == nullptr || a.rowdot2 == nullptr) return "par_qk: the dK operands are missing";
  if (a.stride < 1 || a.stride > kMaxStateStride) return "par_qk: state stride out of range";
  const int MT = par_qk_head_tile(a.DHQK);
  if (MT == 256) return launch_par_qk_pair_t<256>(a, BH, stream);
  if (MT == 128) return launch_par_qk_pair_t<128>(a, BH, stream);
  return launch_par_qk_pair_t<64>(a, BH, stream);
}

}  // namespace mlstm
