// Chunk-parallel kernels whose output tile spans value columns: the forward output H and the gradient dV.
//
// forward (mlstm_kernels/torch/chunkwise/native/fw.py:171-212 in the reference), per chunk:
//   Sbar[t][j] = (q_t . k_j)/sqrt(DHQK) * exp(u_t - w_j)   (j <= t)
//   H[t][:]    = ( bbar_t/sqrt(DHQK) * q_t^T C_prev + sum_j Sbar[t][j] v_j ) / (max(|den_t|, floor_t) + eps)
//   den_t      = bbar_t/sqrt(DHQK) * q_t . n_prev + sum_j Sbar[t][j]
// backward dV (mlstm_kernels/torch/chunkwise/native/bw.py:153-198), per chunk:
//   dV[j][:]   = sum_t Sbar[t][j] rho_t dH[t][:]  +  abar_j * k_j^T dC_next          rho_t = 1/(nrow_t + eps)
//
// Both are the same GEMM chain on a transposed output tile  Out^T[w][n]  (value columns x chunk positions):
//   Out^T = ( State^T[w][d] . Xn^T[d][n] ) * colscale[n]  +  Xw^T[w][o] . P[o][n]
// with  n = query position t, o = key position j, Xn = Q, Xw = V, State = C_prev       (forward)
//       n = key position j,   o = query position t, Xn = K, Xw = dH, State = dC_next   (dV)
//   * State^T arrives as ready-made bf16 MFMA fragments written by the scan kernel (16 B per lane, no LDS),
//   * Xn stays resident in LDS (it feeds the score matrix, the inter-chunk product and, forward, q.n),
//   * colscale multiplies the fp32 accumulator after the inter-chunk product (positions are accumulator
//     columns), so Xn is never rescaled or re-rounded,
//   * the gated score matrix P is produced by the four waves cooperatively (fp32 gating, bf16 into LDS),
//   * Xw^T fragments come from row-major slabs through the transposing LDS read.
// Four waves form a 2 x 2 grid over (value columns, positions); each wave owns (WT/2) x 64 outputs.
#include "common.h"
#include "kernels.h"

namespace mlstm {

template <int WT, bool IS_DV>
__global__ __launch_bounds__(256) void par_hv_kernel(ParHvArgs a) {
  constexpr int MB = WT / 64;   // 32-row value blocks per wave
  constexpr int PS = 128 + 8;   // score matrix row stride: P stored as Pn[n][o]
  constexpr int KS = 64 + 8;    // slab row stride of the streamed score operand
  constexpr int VS = WT + 16;   // slab row stride of the streamed value-side operand
  constexpr int HS = WT + 8;    // output staging row stride
  const int DHQK = a.DHQK, DHHV = a.DHHV, S = a.S, NC = a.NC;
  const int QS = DHQK + 8;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  const int n_region = 128 * (QS > HS ? QS : HS);
  uint16_t* Ns = (uint16_t*)smem_raw;  // resident Xn tile [128][DHQK] in fragment order
  uint16_t* Ps = Ns + n_region;
  uint16_t* Ts = Ps + 128 * PS;
  constexpr int t_region = (128 * KS > 32 * VS) ? 128 * KS : 32 * VS;
  float* uu = (float*)(Ts + t_region);
  float* ww = uu + 128;
  float* cs = ww + 128;       // column scale
  float* inv = cs + 128;      // forward: 1/(nmax + eps); dV: rho_t
  float* rows = inv + 128;    // [2][128] partial row sums of Sbar (forward)
  float* nperm = rows + 256;  // [DHQK] n_prev in fragment order (forward)

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int mi = wave >> 1, ni = wave & 1;
  const int r = lane & 31, h = lane >> 5;
  const BlockId blk = xcd_block_id();  // the column tiles of one chunk share Q, K: keep them on one XCD
  const int bh = blk.z, c = blk.y;
  const int w_tile = blk.x * WT;
  const size_t Sp = (size_t)NC * kChunk;
  const size_t gofs = bh * Sp + (size_t)c * kChunk;
  const int t_base = c * kChunk;
  const uint16_t* Xn_g = (IS_DV ? a.K : a.Q) + (size_t)bh * S * DHQK;  // resident operand
  const uint16_t* Xo_g = (IS_DV ? a.Q : a.K) + (size_t)bh * S * DHQK;  // streamed score operand
  const uint16_t* Xw_g = (IS_DV ? a.dH : a.V) + (size_t)bh * S * DHHV + w_tile;

  // ---- phase 0: resident tile, gate vectors (and n_prev) into LDS
  {
    const int vec_per_row = DHQK / 8;
    for (int idx = tid; idx < 128 * vec_per_row; idx += 256) {
      const int j = idx / vec_per_row, cv = idx % vec_per_row;
      const int t = t_base + j;
      const uint4 v = t < S ? *(const uint4*)(Xn_g + (size_t)t * DHQK + cv * 8) : make_uint4(0, 0, 0, 0);
      store_perm16(Ns + j * QS, cv, v);
    }
    if (tid < 128) {
      uu[tid] = a.g.u[gofs + tid];
      ww[tid] = a.g.w[gofs + tid];
      if (IS_DV) {
        cs[tid] = a.g.abar[gofs + tid];
        inv[tid] = a.use_nrow ? 1.f / (a.nrow[gofs + tid] + a.eps) : 1.f;
      } else {
        cs[tid] = a.g.bbar[gofs + tid] * a.qk_scale;
      }
    }
    if (!IS_DV)
      for (int d = tid; d < DHQK; d += 256) nperm[perm16(d)] = a.nstates[((size_t)bh * NC + c) * DHQK + d];
  }

  // ---- phase S: score quadrant (64 o x 64 n) per wave, contraction over DHQK in slabs of 64
  f32x16 sacc[2][2];
#pragma unroll
  for (int ob = 0; ob < 2; ++ob)
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) sacc[ob][nb][i] = 0.f;
  // quadrant entirely above the diagonal: forward (o = j, n = t): j-half 1, t-half 0; dV (o = t, n = j): t-half 0, j-half 1
  const bool quadrant_live = IS_DV ? !(mi == 0 && ni == 1) : !(mi == 1 && ni == 0);
  for (int slab = 0; slab < DHQK / 64; ++slab) {
    __syncthreads();  // previous slab fully consumed (and phase-0 writes visible on the first pass)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int idx = tid + v * 256;
      const int j = idx >> 3, cv = idx & 7;
      const int t = t_base + j;
      const uint4 kv = t < S ? *(const uint4*)(Xo_g + (size_t)t * DHQK + slab * 64 + cv * 8) : make_uint4(0, 0, 0, 0);
      store_perm16(Ts + j * KS, cv, kv);
    }
    __syncthreads();
    if (quadrant_live) {
#pragma unroll
      for (int ds = 0; ds < 4; ++ds) {
        Frag A[2], B[2];
#pragma unroll
        for (int ob = 0; ob < 2; ++ob) A[ob].u = *(const uint4*)(Ts + (64 * mi + 32 * ob + r) * KS + 16 * ds + 8 * h);
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
          B[nb].u = *(const uint4*)(Ns + (64 * ni + 32 * nb + r) * QS + slab * 64 + 16 * ds + 8 * h);
#pragma unroll
        for (int ob = 0; ob < 2; ++ob)
#pragma unroll
          for (int nb = 0; nb < 2; ++nb) mfma32(sacc[ob][nb], A[ob], B[nb]);
      }
    }
  }
  // gate, mask, round, and write P as Ps[n][o]; forward also accumulates fp32 row sums over j
  {
    float rsum[2] = {0.f, 0.f};
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      const int n = 64 * ni + 32 * nb + r;
      const float un = IS_DV ? ww[n] : uu[n];  // dV: n is the key position j -> w_j ; forward: n = t -> u_t
#pragma unroll
      for (int ob = 0; ob < 2; ++ob) {
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int o0 = 64 * mi + 32 * ob + 8 * g4 + 4 * h;
          const float4 xo = *(const float4*)((IS_DV ? uu : ww) + o0);
          const float xov[4] = {xo.x, xo.y, xo.z, xo.w};
          float rho[4] = {1.f, 1.f, 1.f, 1.f};
          if (IS_DV) {
            const float4 rr = *(const float4*)(inv + o0);
            rho[0] = rr.x; rho[1] = rr.y; rho[2] = rr.z; rho[3] = rr.w;
          }
          float pv[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            // exponent u_t - w_j and causal mask j <= t
            const float ex = IS_DV ? (xov[e] - un) : (un - xov[e]);
            const bool keep = IS_DV ? (n <= o0 + e) : (o0 + e <= n);
            const float val = sacc[ob][nb][4 * g4 + e] * a.qk_scale * __expf(ex) * rho[e];
            pv[e] = keep ? val : 0.f;
            rsum[nb] += pv[e];
          }
          *(uint2*)(Ps + n * PS + o0) = make_uint2(pack_bf16x2(pv[0], pv[1]), pack_bf16x2(pv[2], pv[3]));
        }
      }
    }
    if (!IS_DV) {
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        const float tot = rsum[nb] + __shfl_xor(rsum[nb], 32);
        if (h == 0) rows[mi * 128 + 64 * ni + 32 * nb + r] = tot;
      }
    }
  }
  __syncthreads();

  // ---- phase D (forward): denominators
  if (!IS_DV) {
    const int t = tid >> 1, part = tid & 1;
    const int half = DHQK / 2;
    const uint16_t* qrow = Ns + t * QS + part * half;
    const float* np = nperm + part * half;
    float dot = 0.f;
    for (int d = 0; d < half; d += 8) {
      const uint4 qv = *(const uint4*)(qrow + d);
      const uint32_t qq[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        dot += __uint_as_float(qq[p] << 16) * np[d + 2 * p];
        dot += __uint_as_float(qq[p] & 0xffff0000u) * np[d + 2 * p + 1];
      }
    }
    dot += __shfl_xor(dot, 1);
    if (part == 0) {
      float nmax = 1.f, iv = 1.f;
      if (a.use_nrow) {
        const float den = cs[t] * dot + rows[t] + rows[128 + t];
        const float mc = a.g.mcomb[gofs + t];
        const float floor_v = a.sig_gate ? 1.f : __expf(-mc);
        nmax = fmaxf(fabsf(den), floor_v);
        iv = 1.f / (nmax + a.eps);
      }
      inv[t] = iv;
      if (blk.x == 0) {
        a.nrow_out[gofs + t] = nmax;
        if (t_base + t < S) {
          if (a.n_out != nullptr) a.n_out[(size_t)bh * S + t_base + t] = nmax;
          if (a.m_out != nullptr) a.m_out[(size_t)bh * S + t_base + t] = a.g.mcomb[gofs + t];
        }
      }
    }
  }

  // ---- main phase: Out^T = (State^T Xn^T) * colscale + Xw^T P
  f32x16 acc[MB][2];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.f;
  const int m_wave = mi * (WT / 2);  // first value column of this wave inside the tile
  {
    const size_t ND = DHQK / 16, NW = DHHV / 32;
    const uint4* st = (const uint4*)a.states + ((size_t)bh * NC + c) * NW * ND * 64;
    const size_t W32 = (size_t)(w_tile + m_wave) / 32;
    for (int ds = 0; ds < (int)ND; ++ds) {
      Frag A[MB], B[2];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) A[mb].u = st[((W32 + mb) * ND + ds) * 64 + lane];
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) B[nb].u = *(const uint4*)(Ns + (64 * ni + 32 * nb + r) * QS + 16 * ds + 8 * h);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) mfma32(acc[mb][nb], A[mb], B[nb]);
    }
  }
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const float sc = cs[64 * ni + 32 * nb + r];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb][nb] *= sc;
  }
  {
    const int q16 = (lane >> 4) & 1, i16 = lane & 15;
    const int krow = 8 * h + (i16 >> 2), ncol = 16 * q16 + 4 * (i16 & 3);
    for (int slab = 0; slab < 4; ++slab) {
      __syncthreads();  // previous slab consumed (first pass: P / inv written, score slabs consumed)
      constexpr int vec_per_row = WT / 8;
      for (int idx = tid; idx < 32 * vec_per_row; idx += 256) {
        const int j = idx / vec_per_row, cv = idx % vec_per_row;
        const int t = t_base + slab * 32 + j;
        const uint4 vv = t < S ? *(const uint4*)(Xw_g + (size_t)t * DHHV + cv * 8) : make_uint4(0, 0, 0, 0);
        *(uint4*)(Ts + j * VS + cv * 8) = vv;
      }
      __syncthreads();
      // forward: queries < 64 never see keys >= 64; dV: keys >= 64 are never seen by queries < 64
      if (IS_DV ? (ni == 1 && slab < 2) : (ni == 0 && slab >= 2)) continue;
#pragma unroll
      for (int jl = 0; jl < 2; ++jl) {
        Frag A[MB], B[2];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          const uint16_t* p = Ts + (16 * jl + krow) * VS + (m_wave + 32 * mb + ncol);
          A[mb].d[0] = lds_read_tr16(p);
          A[mb].d[1] = lds_read_tr16(p + 4 * VS);
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
  __syncthreads();  // resident tile no longer needed: its region becomes the output staging tile

  // ---- epilogue: (normalise,) round, transpose through LDS, coalesced store
  uint16_t* Hs = Ns;
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int n = 64 * ni + 32 * nb + r;
    const float iv = IS_DV ? 1.f : inv[n];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int w0 = m_wave + 32 * mb + 8 * g4 + 4 * h;
        *(uint2*)(Hs + n * HS + w0) =
            make_uint2(pack_bf16x2(acc[mb][nb][4 * g4 + 0] * iv, acc[mb][nb][4 * g4 + 1] * iv),
                       pack_bf16x2(acc[mb][nb][4 * g4 + 2] * iv, acc[mb][nb][4 * g4 + 3] * iv));
      }
  }
  __syncthreads();
  {
    uint16_t* Og = a.Out + (size_t)bh * S * DHHV + w_tile;
    constexpr int vec_per_row = WT / 8;
    for (int idx = tid; idx < 128 * vec_per_row; idx += 256) {
      const int j = idx / vec_per_row, cv = idx % vec_per_row;
      const int t = t_base + j;
      if (t < S) *(uint4*)(Og + (size_t)t * DHHV + cv * 8) = *(const uint4*)(Hs + j * HS + cv * 8);
    }
  }
}

template <int WT, bool IS_DV>
static const char* launch_par_hv_t(const ParHvArgs& a, int BH, hipStream_t stream) {
  const int QS = a.DHQK + 8, HS = WT + 8;
  const size_t n_region = (size_t)128 * (QS > HS ? QS : HS);
  const size_t t_region = (128 * 72 > 32 * (WT + 16)) ? 128 * 72 : 32 * (WT + 16);
  const size_t smem = (n_region + 128 * 136 + t_region) * 2 + (size_t)(6 * 128 + a.DHQK) * 4;
  if (smem > 160 * 1024) return "par_hv: DHQK too large for the LDS-resident tile";
  if (hipFuncSetAttribute((const void*)par_hv_kernel<WT, IS_DV>, hipFuncAttributeMaxDynamicSharedMemorySize,
                          (int)smem) != hipSuccess)
    return "par_hv: cannot raise the dynamic LDS limit";
  dim3 grid(a.DHHV / WT, a.NC, BH);
  hipLaunchKernelGGL((par_hv_kernel<WT, IS_DV>), grid, dim3(256), smem, stream, a);
  return nullptr;
}

const char* launch_par_hv(const ParHvArgs& a, int BH, bool is_dv, hipStream_t stream) {
  if (a.DHQK % 64 != 0 || a.DHHV % 64 != 0) return "par_hv: DHQK and DHHV must be multiples of 64";
  if (is_dv) {
    if (a.DHHV % 256 == 0) return launch_par_hv_t<256, true>(a, BH, stream);
    if (a.DHHV % 128 == 0) return launch_par_hv_t<128, true>(a, BH, stream);
    return launch_par_hv_t<64, true>(a, BH, stream);
  }
  if (a.DHHV % 256 == 0) return launch_par_hv_t<256, false>(a, BH, stream);
  if (a.DHHV % 128 == 0) return launch_par_hv_t<128, false>(a, BH, stream);
  return launch_par_hv_t<64, false>(a, BH, stream);
}

}  // namespace mlstm
