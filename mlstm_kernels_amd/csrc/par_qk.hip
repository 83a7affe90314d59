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
// DHHV in slabs of 64 columns feeds BOTH the inter-chunk product and the score matrix from the same Xn slab.
// The state fragments (stored for a contraction over the head dimension) are copied to LDS unchanged and
// re-read with the transposing LDS read, which hands out operands for a contraction over value columns.
// Row sums  sum_d x[n][d] * Out[n][d]  (x = q for dQ, k for dK) are emitted for the gate gradients.
#include "common.h"
#include "kernels.h"

namespace mlstm {

template <int MT, bool IS_DQ>
__global__ __launch_bounds__(256) void par_qk_kernel(ParQkArgs a) {
  constexpr int MB = MT / 64;       // 32-row head-dim blocks per wave
  constexpr int PS = 128 + 8;       // P stored as Ps[n][o]
  constexpr int XS = 64 + 8;        // value-column slab row stride
  constexpr int ZS = MT + 16;       // pass-2 slab row stride
  constexpr int OS = MT + 8;        // output staging row stride
  constexpr int NDT = MT / 16;      // 16-row state fragments per 32 value columns inside the tile
  constexpr int CF = 2 * NDT * 64 * 8;  // elements of the staged state fragments per 64-column slab
  const int DHQK = a.DHQK, DHHV = a.DHHV, S = a.S, NC = a.NC;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  // stage region: [state frags | Xn slab | Xo slab], later pass-2 slabs, later the output staging tile
  constexpr int stage_elems_a = CF + 2 * 128 * XS;
  constexpr int stage_elems_b = 128 * OS;
  constexpr int stage_elems = stage_elems_a > stage_elems_b ? stage_elems_a : stage_elems_b;
  uint16_t* Cf = (uint16_t*)smem_raw;
  uint16_t* Xn = Cf + CF;
  uint16_t* Xo = Xn + 128 * XS;
  uint16_t* Ps = Cf + stage_elems;
  float* uu = (float*)(Ps + 128 * PS);
  float* ww = uu + 128;
  float* cs = ww + 128;    // column scale
  float* rho = cs + 128;   // 1/(nrow + eps)

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int mi = wave >> 1, ni = wave & 1;
  const int r = lane & 31, h = lane >> 5;
  const BlockId blk = xcd_block_id();
  const int bh = blk.z, c = blk.y;
  const int d_tile = blk.x * MT;
  const size_t Sp = (size_t)NC * kChunk;
  const size_t gofs = bh * Sp + (size_t)c * kChunk;
  const int t_base = c * kChunk;
  const uint16_t* Xn_g = (IS_DQ ? a.dH : a.V) + (size_t)bh * S * DHHV;
  const uint16_t* Xo_g = (IS_DQ ? a.V : a.dH) + (size_t)bh * S * DHHV;
  const uint16_t* Z_g = (IS_DQ ? a.K : a.Q) + (size_t)bh * S * DHQK + d_tile;

  if (tid < 128) {
    uu[tid] = a.g.u[gofs + tid];
    ww[tid] = a.g.w[gofs + tid];
    const float rh = a.use_nrow ? 1.f / (a.nrow[gofs + tid] + a.eps) : 1.f;
    rho[tid] = rh;
    cs[tid] = IS_DQ ? a.g.bbar[gofs + tid] * a.qk_scale * rh : a.g.abar[gofs + tid];
  }

  f32x16 acc[MB][2], sacc[2][2];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.f;
#pragma unroll
  for (int ob = 0; ob < 2; ++ob)
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) sacc[ob][nb][i] = 0.f;
  // dQ: o = j, n = t: dead quadrant j-half 1 / t-half 0.  dK: o = t, n = j: dead quadrant t-half 0 / j-half 1.
  const bool quadrant_live = IS_DQ ? !(mi == 1 && ni == 0) : !(mi == 0 && ni == 1);
  const int m_wave = mi * (MT / 2);

  // ---- pass 1 over the value columns
  {
    const size_t ND = DHQK / 16, NW = DHHV / 32;
    const uint4* st = (const uint4*)a.states + ((size_t)bh * NC + c) * NW * ND * 64;
    const int q16 = (lane >> 4) & 1, i16 = lane & 15;
    // transposing read of the staged fragments: lane i16 of a 16-lane block addresses value column
    // k0 + i16/4 and the 4 consecutive head-dim rows n0 + 4*(i16%4) .. +3
    const int d_grp = i16 & 3;                          // which group of 4 rows inside the 16-row fragment
    const int frag_byte = 32 * (d_grp & 1) * 16 + 8 * (d_grp >> 1);  // h_src = d_grp & 1, a_src = d_grp >> 1
    for (int slab = 0; slab < DHHV / 64; ++slab) {
      __syncthreads();
      // state fragments of value blocks 2*slab, 2*slab+1 and head-dim fragments of this tile: contiguous per block
      for (int idx = tid; idx < 2 * NDT * 64; idx += 256) {
        const int wb_l = idx / (NDT * 64), rem = idx % (NDT * 64);
        ((uint4*)Cf)[idx] = st[((size_t)(2 * slab + wb_l) * ND + d_tile / 16) * 64 + rem];
      }
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int idx = tid + v * 256;
        const int j = idx >> 3, cv = idx & 7;
        const int t = t_base + j;
        const bool ok = t < S;
        const size_t go = (size_t)t * DHHV + slab * 64 + cv * 8;
        *(uint4*)(Xn + j * XS + cv * 8) = ok ? *(const uint4*)(Xn_g + go) : make_uint4(0, 0, 0, 0);
        *(uint4*)(Xo + j * XS + cv * 8) = ok ? *(const uint4*)(Xo_g + go) : make_uint4(0, 0, 0, 0);
      }
      __syncthreads();
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        Frag B[2];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) B[nb].u = *(const uint4*)(Xn + (64 * ni + 32 * nb + r) * XS + 16 * ks + 8 * h);
        // inter-chunk product: A = State[d][w]
        {
          Frag A[MB];
          const int wrow = 16 * ks + 8 * h + (i16 >> 2);      // value column inside the slab (first read)
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) {
            const int ds_l = (m_wave + 32 * mb + 16 * q16) / 16;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
              const int wr = wrow + 4 * half;
              const unsigned char* p = (const unsigned char*)Cf + ((size_t)((wr >> 5) * NDT + ds_l) * 64 + (wr & 31)) * 16 + frag_byte;
              A[mb].d[half] = lds_read_tr16(p);
            }
          }
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) mfma32(acc[mb][nb], A[mb], B[nb]);
        }
        // score matrix: A = Xo rows
        if (quadrant_live) {
          Frag A[2];
#pragma unroll
          for (int ob = 0; ob < 2; ++ob) A[ob].u = *(const uint4*)(Xo + (64 * mi + 32 * ob + r) * XS + 16 * ks + 8 * h);
#pragma unroll
          for (int ob = 0; ob < 2; ++ob)
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) mfma32(sacc[ob][nb], A[ob], B[nb]);
        }
      }
    }
  }
  // column scale of the inter-chunk part
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const float sc = cs[64 * ni + 32 * nb + r];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb][nb] *= sc;
  }
  // gate the score matrix: P[o][n] = sacc * exp(u_t - w_j)/sqrt(DHQK) * rho_t for j <= t; store as Ps[n][o]
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int n = 64 * ni + 32 * nb + r;
    const float xn = IS_DQ ? uu[n] : ww[n];
    const float rn = IS_DQ ? rho[n] : 1.f;
#pragma unroll
    for (int ob = 0; ob < 2; ++ob)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int o0 = 64 * mi + 32 * ob + 8 * g4 + 4 * h;
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
          const float val = sacc[ob][nb][4 * g4 + e] * a.qk_scale * __expf(ex) * rn * ro[e];
          pv[e] = keep ? val : 0.f;
        }
        *(uint2*)(Ps + n * PS + o0) = make_uint2(pack_bf16x2(pv[0], pv[1]), pack_bf16x2(pv[2], pv[3]));
      }
  }

  // ---- pass 2 over the chunk positions o: Out^T += Z^T P
  {
    uint16_t* Zs = Cf;
    const int q16 = (lane >> 4) & 1, i16 = lane & 15;
    const int krow = 8 * h + (i16 >> 2), ncol = 16 * q16 + 4 * (i16 & 3);
    for (int slab = 0; slab < 4; ++slab) {
      __syncthreads();  // first pass: P written and pass-1 slabs consumed
      constexpr int vec_per_row = MT / 8;
      for (int idx = tid; idx < 32 * vec_per_row; idx += 256) {
        const int j = idx / vec_per_row, cv = idx % vec_per_row;
        const int t = t_base + slab * 32 + j;
        *(uint4*)(Zs + j * ZS + cv * 8) = t < S ? *(const uint4*)(Z_g + (size_t)t * DHQK + cv * 8) : make_uint4(0, 0, 0, 0);
      }
      __syncthreads();
      // dQ (n = t, o = j <= t): queries < 64 skip key slabs >= 2.  dK (n = j, o = t >= j): keys >= 64 skip query slabs < 2.
      if (IS_DQ ? (ni == 0 && slab >= 2) : (ni == 1 && slab < 2)) continue;
#pragma unroll
      for (int jl = 0; jl < 2; ++jl) {
        Frag A[MB], B[2];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          const uint16_t* p = Zs + (16 * jl + krow) * ZS + (m_wave + 32 * mb + ncol);
          A[mb].d[0] = lds_read_tr16(p);
          A[mb].d[1] = lds_read_tr16(p + 4 * ZS);
        }
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
          B[nb].u = *(const uint4*)(Ps + (64 * ni + 32 * nb + r) * PS + slab * 32 + 16 * jl + 8 * h);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
          for (int nb = 0; nb < 2; ++nb) mfma32(acc[mb][nb], A[mb], B[nb]);
      }
    }
  }
  __syncthreads();

  // ---- epilogue part 1: row dots  sum_d x[n][d] * Out[n][d]  from the fp32 accumulators (x = q for dQ, k for dK).
  // They feed a suffix sum over the whole sequence (dF), where the rounding noise of bf16 outputs would add up
  // like a random walk; the matching x rows are staged in LDS so every lane can read its own row.
  uint16_t* Os = Cf;
  {
    const uint16_t* Rg = (IS_DQ ? a.Q : a.K) + (size_t)bh * S * DHQK + d_tile;
    constexpr int vec_per_row = MT / 8;
    for (int idx = tid; idx < 128 * vec_per_row; idx += 256) {
      const int j = idx / vec_per_row, cv = idx % vec_per_row;
      const int t = t_base + j;
      *(uint4*)(Os + j * OS + cv * 8) = t < S ? *(const uint4*)(Rg + (size_t)t * DHQK + cv * 8) : make_uint4(0, 0, 0, 0);
    }
  }
  __syncthreads();
  float* red = uu;  // [2][128]: uu/ww are dead after the gating step
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int n = 64 * ni + 32 * nb + r;
    float part = 0.f;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int d0 = m_wave + 32 * mb + 8 * g4 + 4 * h;
        const uint2 xv = *(const uint2*)(Os + n * OS + d0);
        part += acc[mb][nb][4 * g4 + 0] * __uint_as_float(xv.x << 16);
        part += acc[mb][nb][4 * g4 + 1] * __uint_as_float(xv.x & 0xffff0000u);
        part += acc[mb][nb][4 * g4 + 2] * __uint_as_float(xv.y << 16);
        part += acc[mb][nb][4 * g4 + 3] * __uint_as_float(xv.y & 0xffff0000u);
      }
    part += __shfl_xor(part, 32);
    if (h == 0) red[mi * 128 + n] = part;
  }
  __syncthreads();
  if (tid < 128) {
    const float dot = red[tid] + red[128 + tid];
    if (gridDim.x == 1) a.rowdot[gofs + tid] = dot;
    else atomicAdd(a.rowdot + gofs + tid, dot);
  }

  // ---- epilogue part 2: round, transpose through LDS, coalesced store
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int n = 64 * ni + 32 * nb + r;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int d0 = m_wave + 32 * mb + 8 * g4 + 4 * h;
        *(uint2*)(Os + n * OS + d0) = make_uint2(pack_bf16x2(acc[mb][nb][4 * g4 + 0], acc[mb][nb][4 * g4 + 1]),
                                                 pack_bf16x2(acc[mb][nb][4 * g4 + 2], acc[mb][nb][4 * g4 + 3]));
      }
  }
  __syncthreads();
  {
    uint16_t* Og = a.Out + (size_t)bh * S * DHQK + d_tile;
    constexpr int vec_per_row = MT / 8;
    for (int idx = tid; idx < 128 * vec_per_row; idx += 256) {
      const int j = idx / vec_per_row, cv = idx % vec_per_row;
      const int t = t_base + j;
      if (t < S) *(uint4*)(Og + (size_t)t * DHQK + cv * 8) = *(const uint4*)(Os + j * OS + cv * 8);
    }
  }
}

template <int MT, bool IS_DQ>
static const char* launch_par_qk_t(const ParQkArgs& a, int BH, hipStream_t stream) {
  constexpr int CF = 2 * (MT / 16) * 64 * 8;
  constexpr int sa = CF + 2 * 128 * 72, sb = 128 * (MT + 8);
  const size_t smem = (size_t)((sa > sb ? sa : sb) + 128 * 136) * 2 + 4 * 128 * 4;
  if (hipFuncSetAttribute((const void*)par_qk_kernel<MT, IS_DQ>, hipFuncAttributeMaxDynamicSharedMemorySize,
                          (int)smem) != hipSuccess)
    return "par_qk: cannot raise the dynamic LDS limit";
  dim3 grid(a.DHQK / MT, a.NC, BH);
  hipLaunchKernelGGL((par_qk_kernel<MT, IS_DQ>), grid, dim3(256), smem, stream, a);
  return nullptr;
}

const char* launch_par_qk(const ParQkArgs& a, int BH, bool is_dq, hipStream_t stream) {
  if (a.DHQK % 64 != 0 || a.DHHV % 64 != 0) return "par_qk: DHQK and DHHV must be multiples of 64";
  if (is_dq) {
    if (a.DHQK % 256 == 0) return launch_par_qk_t<256, true>(a, BH, stream);
    if (a.DHQK % 128 == 0) return launch_par_qk_t<128, true>(a, BH, stream);
    return launch_par_qk_t<64, true>(a, BH, stream);
  }
  if (a.DHQK % 256 == 0) return launch_par_qk_t<256, false>(a, BH, stream);
  if (a.DHQK % 128 == 0) return launch_par_qk_t<128, false>(a, BH, stream);
  return launch_par_qk_t<64, false>(a, BH, stream);
}

}  // namespace mlstm
