// Chunk-parallel backward kernels whose output tile spans the query/key head dimension: dQ and dK.
//
// (mlstm_kernels/torch/chunkwise/native/bw.py:153-198 in the reference), per chunk, rho_t = 1/(nrow_t + eps):
//   dS[t][j] = exp(u_t - w_j)/sqrt(DHQK) * rho_t * (dH_t . v_j)                                (j <= t)
//   dQ[t][:] = sum_j dS[t][j] k_j  +  bbar_t/sqrt(DHQK) * rho_t * C_prev dH_t
//   dK[j][:] = sum_t dS[t][j] q_t  +  abar_j * dC_next v_j
//
// Both are one GEMM chain on the transposed output tile  Out^T[d][n]  (head dimension x chunk positions):
//   Out^T = ( State[d][w] . Xn^T[w][n] ) * colscale[n]  +  Z^T[d][o] . P[o][n]
// with  n = t, o = j, Xn = dH, Xo = V,  Z = K, State = C_prev    (dQ)
//       n = j, o = t, Xn = V,  Xo = dH, Z = Q, State = dC_next   (dK)
// and the score matrix  P[o][n] = gate * (Xo Xn^T)  contracted over the DHHV value columns.  One pass over
// DHHV in slabs of 32 columns feeds BOTH the inter-chunk product and the score matrix from the same Xn slab.
// The state fragments (stored for a contraction over the head dimension) are copied to LDS unchanged and
// re-read with the transposing LDS read, which hands out operands for a contraction over value columns.
// Row sums  sum_d x[n][d] * Out[n][d]  (x = q for dQ, k for dK) are emitted for the gate gradients.
//
// A workgroup owns MT head-dim rows x 64 positions (half a chunk); two slabs are in flight from global memory into
// registers while a third is being multiplied, and the footprint (54 KB of LDS) lets two workgroups share a CU so
// that one computes while the other waits for memory.  dQ and dK run as ONE launch (par_qk_pair_kernel).
//
// Measured on MI355X at B=4, S=16384, 256/512 and not kept: eight waves of 32 head-dim rows per workgroup (four
// waves per SIMD; 0.99 ms against 0.97 ms for the pair launch); dV's workgroups in the same launch as well (1.56 ms
// against 1.52 ms for dV followed by the pair launch: they stream the shared operands in another order); the Xo score
// operands fetched straight from global memory in fragment layout instead of through LDS (1.03 against 0.98 ms: 32-byte
// row pieces per lane pair are a poor access pattern, the LDS detour is cheaper).
#include "common.h"
#include "kernels.h"

namespace mlstm {

template <int MT, bool IS_DQ>
__device__ __forceinline__ void par_qk_body(const ParQkArgs& a, const BlockId blk) {
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
  float* uu = (float*)(Ps + 64 * PS);  // [128]
  float* ww = uu + 128;                // [128]
  float* rho = ww + 128;               // [128] 1/(nrow + eps)
  float* cs = rho + 128;               // [64] column scale of this workgroup's positions
  float* red = cs + 64;                // [NWAVE][64] row-dot partials

  // the wave index is made scalar so that branches on it are scalar branches (accumulators stay in place)
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, h = lane >> 5;
#ifdef MLSTM_PAR_TIMING
  unsigned long long tph[7] = {0, 0, 0, 0, 0, 0, 0}, tlast = __builtin_amdgcn_s_memtime();
  const unsigned long long tstart = tlast;
#define MLSTM_PTICK(p_) { const unsigned long long now_ = __builtin_amdgcn_s_memtime(); tph[p_] += now_ - tlast; tlast = now_; }
#else
#define MLSTM_PTICK(p_)
#endif
  const int bh = blk.z, c = blk.y;
  const int nh = blk.x & 1;
  const int d_tile = (blk.x >> 1) * MT;
  const size_t Sp = (size_t)NC * kChunk;
  const size_t gofs = bh * Sp + (size_t)c * kChunk;
  const int t_base = c * kChunk;
  const int n0 = 64 * nh;
  // live 32-row blocks of the other position index: dQ o = j <= t, dK o = t >= j
  const int ob_lo = IS_DQ ? 0 : 2 * nh, ob_hi = IS_DQ ? 2 * (nh + 1) : 4;
  const uint16_t* Xn_g = (IS_DQ ? a.dH : a.V) + (size_t)bh * S * DHHV;
  const uint16_t* Xo_g = (IS_DQ ? a.V : a.dH) + (size_t)bh * S * DHHV;
  const uint16_t* Z_g = (IS_DQ ? a.K : a.Q) + (size_t)bh * S * DHQK + d_tile;

  for (int idx = tid; idx < 128; idx += NTH) {
    uu[idx] = a.g.u[gofs + idx];
    ww[idx] = a.g.w[gofs + idx];
    rho[idx] = a.use_nrow ? 1.f / (a.nrow[gofs + idx] + a.eps) : 1.f;
  }
  for (int idx = tid; idx < 64; idx += NTH) {
    const float rh = a.use_nrow ? 1.f / (a.nrow[gofs + n0 + idx] + a.eps) : 1.f;
    cs[idx] = IS_DQ ? a.g.bbar[gofs + n0 + idx] * a.qk_scale * rh : a.g.abar[gofs + n0 + idx];
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

  // ---- pass 1 over the value columns
  {
    const size_t ND = DHQK / 16, NW = DHHV / 32;
    const u32x4* st = (const u32x4*)a.states + ((size_t)bh * NC + c) * NW * ND * 64;
    constexpr int CV = NDT * 64 / NTH;      // state-fragment vectors per thread per slab
    // The state fragments come in slabs of 32 value columns, two slabs in flight in registers.  The Xn / Xo rows are
    // fetched 64 columns at a time (one fetch serves two state slabs): 128 contiguous bytes per row and load
    // instruction instead of 64.
    constexpr int NV = 64 * 8 / NTH;        // Xn vectors per thread per pair of slabs
    constexpr int OV = 128 * 8 / NTH;       // Xo vectors per thread per pair of slabs
    u32x4 cregA[CV], cregB[CV];
    uint4 nreg[NV], oreg[OV];
    // (macros, not lambdas: with the arrays captured by reference the compiler kept them in scratch memory)
#define MLSTM_LOAD_C(slab_, creg)                                                                                    \
  {                                                                                                                  \
    _Pragma("unroll") for (int v = 0; v < CV; ++v)                                                                   \
        creg[v] = st[((size_t)(slab_) * ND + d_tile / 16) * 64 + tid + v * NTH];                                     \
  }
#define MLSTM_LOAD_X(pair_)                                                                                          \
  {                                                                                                                  \
    _Pragma("unroll") for (int v = 0; v < NV; ++v) {                                                                 \
      const int idx = tid + v * NTH;                                                                                 \
      const int t = t_base + n0 + (idx >> 3);                                                                        \
      nreg[v] = t < S ? *(const uint4*)(Xn_g + (size_t)t * DHHV + (pair_) * 64 + (idx & 7) * 8) : make_uint4(0, 0, 0, 0); \
    }                                                                                                                \
    _Pragma("unroll") for (int v = 0; v < OV; ++v) {                                                                 \
      const int idx = tid + v * NTH;                                                                                 \
      const int j = idx >> 3;                                                                                        \
      const int t = t_base + j;                                                                                      \
      const bool live = j >= 32 * ob_lo && j < 32 * ob_hi && t < S;                                                  \
      oreg[v] = live ? *(const uint4*)(Xo_g + (size_t)t * DHHV + (pair_) * 64 + (idx & 7) * 8) : make_uint4(0, 0, 0, 0); \
    }                                                                                                                \
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
    const int q16 = (lane >> 4) & 1, i16 = lane & 15;
    // transposing read of the staged fragments: lane i16 of a 16-lane block addresses value column
    // k0 + i16/4 and the 4 consecutive head-dim rows n0 + 4*(i16%4) .. +3
    const int d_grp = i16 & 3;
    const int h_src = d_grp & 1, a_src = d_grp >> 1;
    const int nslab = DHHV / 32;  // even: DHHV is a multiple of 64
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
              const int slot = (32 * h_src + wr) ^ (h_src << 2);
              const unsigned char* p = (const unsigned char*)Cf + ((size_t)ds_l * 64 + slot) * 16 + 8 * a_src;
              A[mb].d[half] = lds_read_tr16(p);
            }
          }
#pragma unroll
          for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) mfma32(acc[mb][nb], A[mb], B[nb]);
        }
        // score matrix: A = Xo rows of the blocks dealt to this wave
#pragma unroll
        for (int k = 0; k < OBW; ++k) {
          // unconditional on purpose: a wave whose block lies above the diagonal multiplies zero rows (its result
          // is dropped at the gating step); a branch here would make the compiler shuttle the score accumulators
          // between the two register files on every iteration
          const int ob = ob_lo + wave + k * NWAVE;
          const int obc = ob < 4 ? ob : 3;
          Frag A;
          A.u = *(const uint4*)(Xo + (32 * obc + r) * XS + 32 * sub + 16 * ks + 8 * h);
#pragma unroll
          for (int nb = 0; nb < 2; ++nb) mfma32(sacc[k][nb], A, B[nb]);
        }
      }
    };
    // two state slabs and one Xn / Xo pair are in flight in registers while a slab is multiplied: one memory round
    // trip spans two slab periods.  The prefetches are unconditional (the last iterations re-fetch the last slab): a
    // conditional prefetch makes the compiler keep the prefetch registers in scratch memory across the loop back-edge.
    MLSTM_LOAD_C(0, cregA)
    MLSTM_LOAD_X(0)
    MLSTM_LOAD_C(1, cregB)
    MLSTM_PTICK(0)
    for (int slab = 0; slab < nslab; slab += 2) {
      __syncthreads();
      MLSTM_STORE_C(cregA)
      MLSTM_STORE_X
      __syncthreads();
      MLSTM_LOAD_C(slab + 2 < nslab ? slab + 2 : nslab - 1, cregA)
      MLSTM_LOAD_X(slab + 2 < nslab ? slab / 2 + 1 : slab / 2)
      multiply_slab(0);
      __syncthreads();
      MLSTM_STORE_C(cregB)
      __syncthreads();
      MLSTM_LOAD_C(slab + 3 < nslab ? slab + 3 : nslab - 1, cregB)
      multiply_slab(1);
    }
  }
#undef MLSTM_STORE_C
#undef MLSTM_STORE_X
#undef MLSTM_LOAD_C
#undef MLSTM_LOAD_X
  MLSTM_PTICK(1)
  // column scale of the inter-chunk part
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const float sc = cs[32 * nb + r];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) acc[mb][nb] *= sc;
  }
  // first pass-2 slab (64 positions: two score blocks; the live range is always an even number of blocks) into
  // registers while the score matrix is gated
  constexpr int ZV = 64 * (MT / 8) / NTH;
  uint4 zreg[ZV];
  auto load_zslab = [&](int ob) {
#pragma unroll
    for (int v = 0; v < ZV; ++v) {
      const int idx = tid + v * NTH;
      const int j = idx / (MT / 8), cv = idx % (MT / 8);
      const int t = t_base + 32 * ob + j;
      zreg[v] = t < S ? *(const uint4*)(Z_g + (size_t)t * DHQK + cv * 8) : make_uint4(0, 0, 0, 0);
    }
  };
  load_zslab(ob_lo);
  // the x rows of the row dots (q for dQ, k for dK) are fetched now and parked in registers: their memory round
  // trip overlaps the gating and pass 2 instead of standing alone in the epilogue
  constexpr int XV = 64 * (MT / 8) / NTH;
  uint4 xreg[XV];
  {
    const uint16_t* Rg = (IS_DQ ? a.Q : a.K) + (size_t)bh * S * DHQK + d_tile;
#pragma unroll
    for (int v = 0; v < XV; ++v) {
      const int idx = tid + v * NTH;
      const int j = idx / (MT / 8), cv = idx % (MT / 8);
      const int t = t_base + n0 + j;
      xreg[v] = t < S ? *(const uint4*)(Rg + (size_t)t * DHQK + cv * 8) : make_uint4(0, 0, 0, 0);
    }
  }
  // gate the score matrix: P[o][n] = sacc * exp(u_t - w_j)/sqrt(DHQK) * rho_t for j <= t; store as Ps[n][o]
#pragma unroll
  for (int k = 0; k < OBW; ++k) {
    const int ob = ob_lo + wave + k * NWAVE;
    if (ob < ob_hi) {
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        const int nl = 32 * nb + r;
        const int n = n0 + nl;
        const float xn = IS_DQ ? uu[n] : ww[n];
        const float rn = IS_DQ ? rho[n] : 1.f;
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int o0 = 32 * ob + 8 * g4 + 4 * h;
          const float4 xo = *(const float4*)((IS_DQ ? ww : uu) + o0);
          const float xov[4] = {xo.x, xo.y, xo.z, xo.w};
          float ro[4] = {1.f, 1.f, 1.f, 1.f};
          if (!IS_DQ) {
            const float4 rr = *(const float4*)(rho + o0);
            ro[0] = rr.x; ro[1] = rr.y; ro[2] = rr.z; ro[3] = rr.w;
          }
          float pv[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float ex = IS_DQ ? (xn - xov[e]) : (xov[e] - xn);
            const bool keep = IS_DQ ? (o0 + e <= n) : (n <= o0 + e);
            const float val = sacc[k][nb][4 * g4 + e] * a.qk_scale * __expf(ex) * rn * ro[e];
            pv[e] = keep ? val : 0.f;
          }
          *(uint2*)(Ps + nl * PS + o0) = make_uint2(pack_bf16x2(pv[0], pv[1]), pack_bf16x2(pv[2], pv[3]));
        }
      }
    }
  }

  MLSTM_PTICK(2)
  // ---- pass 2 over the live chunk positions o: Out^T += Z^T P
  {
    uint16_t* Zs = Cf;
    const int q16 = (lane >> 4) & 1, i16 = lane & 15;
    const int krow = 8 * h + (i16 >> 2), ncol = 16 * q16 + 4 * (i16 & 3);
    for (int ob = ob_lo; ob < ob_hi; ob += 2) {
      __syncthreads();  // first pass: P written and pass-1 slabs consumed
#pragma unroll
      for (int v = 0; v < ZV; ++v) {
        const int idx = tid + v * NTH;
        *(uint4*)(Zs + (idx / (MT / 8)) * ZS + (idx % (MT / 8)) * 8) = zreg[v];
      }
      __syncthreads();
      if (ob + 2 < ob_hi) load_zslab(ob + 2);
#pragma unroll
      for (int jl = 0; jl < 4; ++jl) {
        Frag A[2], B[2];
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) {
          const uint16_t* p = Zs + (16 * jl + krow) * ZS + (m_wave + 32 * mb + ncol);
          A[mb].d[0] = lds_read_tr16(p);
          A[mb].d[1] = lds_read_tr16(p + 4 * ZS);
        }
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) B[nb].u = *(const uint4*)(Ps + (32 * nb + r) * PS + 32 * ob + 16 * jl + 8 * h);
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
          for (int nb = 0; nb < 2; ++nb) mfma32(acc[mb][nb], A[mb], B[nb]);
      }
    }
  }
  __syncthreads();

  MLSTM_PTICK(3)
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
        part += acc[mb][nb][4 * g4 + 0] * __uint_as_float(xv.x << 16);
        part += acc[mb][nb][4 * g4 + 1] * __uint_as_float(xv.x & 0xffff0000u);
        part += acc[mb][nb][4 * g4 + 2] * __uint_as_float(xv.y << 16);
        part += acc[mb][nb][4 * g4 + 3] * __uint_as_float(xv.y & 0xffff0000u);
      }
    part += __shfl_xor(part, 32);
    if (h == 0) red[wave * 64 + nl] = part;
  }
  __syncthreads();
  if (tid < 64) {
    float dot = 0.f;
#pragma unroll
    for (int w = 0; w < NWAVE; ++w) dot += red[w * 64 + tid];
    if (DHQK == MT) a.rowdot[gofs + n0 + tid] = dot;
    else atomicAdd(a.rowdot + gofs + n0 + tid, dot);
  }

  MLSTM_PTICK(4)
  // ---- epilogue part 2: round, transpose through LDS, coalesced store
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int nl = 32 * nb + r;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int d0 = m_wave + 32 * mb + 8 * g4 + 4 * h;
        *(uint2*)(Os + nl * OS + d0) = make_uint2(pack_bf16x2(acc[mb][nb][4 * g4 + 0], acc[mb][nb][4 * g4 + 1]),
                                                  pack_bf16x2(acc[mb][nb][4 * g4 + 2], acc[mb][nb][4 * g4 + 3]));
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
  MLSTM_PTICK(5)
#ifdef MLSTM_PAR_TIMING
  if (blk.y == a.NC / 2 && blk.z == 0 && lane == 0)
    for (int p = 0; p < 6; ++p) a.timing[((blk.x + (IS_DQ ? 0 : 2)) * 4 + (wave & 3)) * 8 + p] = tph[p];
  if (tid == 0) {
    const size_t wg = ((size_t)blk.z * a.NC + blk.y) * 2 + blk.x + (IS_DQ ? 0 : 8192);
    a.timing[64 + wg * 2] = tstart;
    a.timing[64 + wg * 2 + 1] = __builtin_amdgcn_s_memtime();
  }
#endif
}

#define PAR_QK_WPE(MT_) ((MT_) == 256 ? 2 : 1)
// dQ and dK of every chunk in ONE launch: the workgroups of a chunk (both gradients, both position halves, all
// head-dimension tiles) are neighbours in launch order and run on the same XCD at about the same time, so the Q, K, V
// and dH rows they all stream are fetched from HBM once and served to the others from the caches.
template <int MT>
__global__ __launch_bounds__(MT) __attribute__((amdgpu_waves_per_eu(PAR_QK_WPE(MT), PAR_QK_WPE(MT)))) void par_qk_pair_kernel(ParQkArgs a) {
  BlockId blk = xcd_block_id();
  const int per = 2 * (a.DHQK / MT);
  if (blk.x < per) {
    par_qk_body<MT, true>(a, blk);
  } else {
    blk.x -= per;
    a.states = a.states2;
    a.Out = a.Out2;
    a.rowdot = a.rowdot2;
    par_qk_body<MT, false>(a, blk);
  }
}

template <int MT>
static const char* launch_par_qk_pair_t(const ParQkArgs& a, int BH, hipStream_t stream) {
  constexpr int CF = (MT / 16) * 64 * 8;
  constexpr int sa = CF + 64 * 72 + 128 * 72, sb = 64 * (MT + 8), sc = 64 * (MT + 32);
  constexpr int sab = sa > sb ? sa : sb;
  constexpr int stage = sab > sc ? sab : sc;
  const size_t smem = (size_t)(stage + 64 * 136) * 2 + (size_t)(3 * 128 + 64 + (MT / 64) * 64) * 4;
  if (hipFuncSetAttribute((const void*)par_qk_pair_kernel<MT>, hipFuncAttributeMaxDynamicSharedMemorySize,
                          (int)smem) != hipSuccess)
    return "par_qk: cannot raise the dynamic LDS limit";
  dim3 grid(4 * (a.DHQK / MT), a.NC, BH);
  hipLaunchKernelGGL((par_qk_pair_kernel<MT>), grid, dim3(MT), smem, stream, a);
  return nullptr;
}

const char* launch_par_qk_pair(const ParQkArgs& a, int BH, hipStream_t stream) {
  if (a.DHQK % 64 != 0 || a.DHHV % 64 != 0) return "par_qk: DHQK and DHHV must be multiples of 64";
  if (a.states2 == nullptr || a.Out2 == nullptr || a.rowdot2 == nullptr) return "par_qk: the dK operands are missing";
  if (a.DHQK % 256 == 0) return launch_par_qk_pair_t<256>(a, BH, stream);
  if (a.DHQK % 128 == 0) return launch_par_qk_pair_t<128>(a, BH, stream);
  return launch_par_qk_pair_t<64>(a, BH, stream);
}

}  // namespace mlstm
