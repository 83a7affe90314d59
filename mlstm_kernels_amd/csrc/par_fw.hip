// Chunk-parallel forward of the TFLA mLSTM: per (batch, head, chunk, slice of value columns)
//
//   Sbar[t][j] = (q_t . k_j) / sqrt(DHQK) * exp(u_t - w_j)            j <= t  (0 above the diagonal)
//   Num[t][:]  = bbar_t / sqrt(DHQK) * q_t^T C_prev  +  sum_j Sbar[t][j] v_j
//   den_t      = bbar_t / sqrt(DHQK) * q_t . n_prev  +  sum_j Sbar[t][j]
//   H[t][:]    = Num[t][:] / (max(|den_t|, floor_t) + eps)            floor = exp(-m_comb) | 1 (sig gate)
//
// (mlstm_kernels/torch/chunkwise/native/fw.py:171-212 in the reference.)  The kernel computes the transposed
// output tile Num^T (value columns x chunk positions) as one GEMM chain whose "weights" are [C_prev^T | V^T]
// and whose "activations" are [Q^T ; Sbar^T]:
//   * C_prev^T arrives as ready-made bf16 MFMA fragments written by the scan kernel (16 B per lane, no LDS),
//   * Q stays resident in LDS for the whole workgroup (it feeds Q K^T, q.n and the inter-chunk product),
//   * the per-row factor bbar_t/sqrt(DHQK) multiplies the fp32 accumulator after the inter-chunk product
//     (positions are accumulator columns), so Q itself is never rescaled or re-rounded,
//   * Sbar is produced by the four waves cooperatively, gated in fp32, rounded to bf16 into LDS,
//   * V^T fragments come from a row-major V slab through the transposing LDS read.
// Four waves form a 2 x 2 grid over (value columns, positions); each wave owns (WT/2) x 64 outputs.
#include "common.h"
#include "kernels.h"

namespace mlstm {


// LDS write of one 16-byte global vector (8 consecutive head-dim entries) in the fragment order used for
// every contraction over DHQK: inside each group of 16, entry 8a + 4h + c is stored at 8h + 4a + c.
__device__ __forceinline__ void store_perm16(uint16_t* row, int cv, uint4 v) {
  const int s16 = (cv >> 1) * 16, a = cv & 1;
  *(uint2*)(row + s16 + 4 * a) = make_uint2(v.x, v.y);
  *(uint2*)(row + s16 + 8 + 4 * a) = make_uint2(v.z, v.w);
}
__device__ __forceinline__ int perm16(int d) {  // position of head-dim entry d in fragment order
  const int s16 = d & ~15, a = (d >> 3) & 1, hh = (d >> 2) & 1, c = d & 3;
  return s16 + 8 * hh + 4 * a + c;
}

template <int WT>
__global__ __launch_bounds__(256) void par_fw_kernel(ParFwArgs a) {
  constexpr int MB = WT / 64;   // 32-row value blocks per wave
  constexpr int PS = 128 + 8;   // Sbar^T row stride
  constexpr int KS = 64 + 8;    // K slab row stride
  constexpr int VS = WT + 16;   // V slab row stride
  constexpr int HS = WT + 8;    // output staging row stride
  const int DHQK = a.DHQK, DHHV = a.DHHV, S = a.S, NC = a.NC;
  const int QS = DHQK + 8;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  const int q_region = 128 * (QS > HS ? QS : HS);
  uint16_t* Qs = (uint16_t*)smem_raw;
  uint16_t* Ps = Qs + q_region;
  uint16_t* Ts = Ps + 128 * PS;
  constexpr int t_region = (128 * KS > 32 * VS) ? 128 * KS : 32 * VS;
  float* uu = (float*)(Ts + t_region);
  float* ww = uu + 128;
  float* cs = ww + 128;       // bbar / sqrt(DHQK)
  float* inv = cs + 128;      // 1 / (nmax + eps)
  float* rows = inv + 128;    // [2][128] partial row sums of Sbar
  float* nperm = rows + 256;  // [DHQK] n_prev in fragment order

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int mi = wave >> 1, ni = wave & 1;
  const int r = lane & 31, h = lane >> 5;
  const int bh = blockIdx.z, c = blockIdx.y;
  const int w_tile = blockIdx.x * WT;
  const size_t Sp = (size_t)NC * kChunk;
  const size_t gofs = bh * Sp + (size_t)c * kChunk;
  const int t_base = c * kChunk;

  // ---- phase 0: Q tile, gate vectors, n_prev into LDS
  {
    const uint16_t* Qg = a.Q + (size_t)bh * S * DHQK;
    const int vec_per_row = DHQK / 8;
    for (int idx = tid; idx < 128 * vec_per_row; idx += 256) {
      const int j = idx / vec_per_row, cv = idx % vec_per_row;
      const int t = t_base + j;
      const uint4 v = t < S ? *(const uint4*)(Qg + (size_t)t * DHQK + cv * 8) : make_uint4(0, 0, 0, 0);
      store_perm16(Qs + j * QS, cv, v);
    }
    if (tid < 128) {
      uu[tid] = a.g.u[gofs + tid];
      ww[tid] = a.g.w[gofs + tid];
      cs[tid] = a.g.bbar[gofs + tid] * a.qk_scale;
    }
    for (int d = tid; d < DHQK; d += 256) nperm[perm16(d)] = a.nstates[((size_t)bh * NC + c) * DHQK + d];
  }

  // ---- phase S: Sbar^T quadrant (64 j x 64 t) per wave, contraction over DHQK in slabs of 64
  f32x16 sacc[2][2];
#pragma unroll
  for (int jb = 0; jb < 2; ++jb)
#pragma unroll
    for (int tb = 0; tb < 2; ++tb)
#pragma unroll
      for (int i = 0; i < 16; ++i) sacc[jb][tb][i] = 0.f;
  const bool quadrant_live = !(mi == 1 && ni == 0);
  {
    const uint16_t* Kg = a.K + (size_t)bh * S * DHQK;
    for (int slab = 0; slab < DHQK / 64; ++slab) {
      __syncthreads();  // previous slab fully consumed (and phase-0 writes visible on the first pass)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int idx = tid + v * 256;
        const int j = idx >> 3, cv = idx & 7;
        const int t = t_base + j;
        const uint4 kv = t < S ? *(const uint4*)(Kg + (size_t)t * DHQK + slab * 64 + cv * 8) : make_uint4(0, 0, 0, 0);
        store_perm16(Ts + j * KS, cv, kv);
      }
      __syncthreads();
      if (quadrant_live) {
#pragma unroll
        for (int ds = 0; ds < 4; ++ds) {
          Frag A[2], B[2];
#pragma unroll
          for (int jb = 0; jb < 2; ++jb) A[jb].u = *(const uint4*)(Ts + (64 * mi + 32 * jb + r) * KS + 16 * ds + 8 * h);
#pragma unroll
          for (int tb = 0; tb < 2; ++tb)
            B[tb].u = *(const uint4*)(Qs + (64 * ni + 32 * tb + r) * QS + slab * 64 + 16 * ds + 8 * h);
#pragma unroll
          for (int jb = 0; jb < 2; ++jb)
#pragma unroll
            for (int tb = 0; tb < 2; ++tb) mfma32(sacc[jb][tb], A[jb], B[tb]);
        }
      }
    }
  }
  // gate, mask, round, and write Sbar^T as Ps[t][j]; accumulate fp32 row sums
  {
    float rsum[2] = {0.f, 0.f};
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) {
      const int t = 64 * ni + 32 * tb + r;
      const float ut = uu[t];
#pragma unroll
      for (int jb = 0; jb < 2; ++jb) {
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int j0 = 64 * mi + 32 * jb + 8 * g4 + 4 * h;
          const float4 wj = *(const float4*)(ww + j0);
          const float wjv[4] = {wj.x, wj.y, wj.z, wj.w};
          float pv[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float val = sacc[jb][tb][4 * g4 + e] * a.qk_scale * __expf(ut - wjv[e]);
            pv[e] = (j0 + e <= t) ? val : 0.f;
            rsum[tb] += pv[e];
          }
          *(uint2*)(Ps + t * PS + j0) = make_uint2(pack_bf16x2(pv[0], pv[1]), pack_bf16x2(pv[2], pv[3]));
        }
      }
    }
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) {
      const float tot = rsum[tb] + __shfl_xor(rsum[tb], 32);
      if (h == 0) rows[mi * 128 + 64 * ni + 32 * tb + r] = tot;
    }
  }
  __syncthreads();

  // ---- phase D: denominators
  {
    const int t = tid >> 1, part = tid & 1;
    const int half = DHQK / 2;
    const uint16_t* qrow = Qs + t * QS + part * half;
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
      if (!(a.sig_gate && !a.normalize)) {
        const float den = cs[t] * dot + rows[t] + rows[128 + t];
        const float mc = a.g.mcomb[gofs + t];
        const float floor_v = a.sig_gate ? 1.f : __expf(-mc);
        nmax = fmaxf(fabsf(den), floor_v);
        iv = 1.f / (nmax + a.eps);
      }
      inv[t] = iv;
      if (blockIdx.x == 0) {
        a.nrow[gofs + t] = nmax;
        if (t_base + t < S) {
          if (a.n_out != nullptr) a.n_out[(size_t)bh * S + t_base + t] = nmax;
          if (a.m_out != nullptr) a.m_out[(size_t)bh * S + t_base + t] = a.g.mcomb[gofs + t];
        }
      }
    }
  }

  // ---- main phase: Num^T = (C_prev^T Q^T) * colscale + V^T Sbar^T
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
    const uint4* st = (const uint4*)a.cstates + ((size_t)bh * NC + c) * NW * ND * 64;
    const size_t W32 = (size_t)(w_tile + m_wave) / 32;
    for (int ds = 0; ds < (int)ND; ++ds) {
      Frag A[MB], B[2];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) A[mb].u = st[((W32 + mb) * ND + ds) * 64 + lane];
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) B[nb].u = *(const uint4*)(Qs + (64 * ni + 32 * nb + r) * QS + 16 * ds + 8 * h);
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
    const uint16_t* Vg = a.V + (size_t)bh * S * DHHV + w_tile;
    const int q16 = (lane >> 4) & 1, i16 = lane & 15;
    const int krow = 8 * h + (i16 >> 2), ncol = 16 * q16 + 4 * (i16 & 3);
    for (int slab = 0; slab < 4; ++slab) {
      __syncthreads();  // previous slab consumed (first pass: Sbar / inv written, K slabs consumed)
      constexpr int vec_per_row = WT / 8;
      for (int idx = tid; idx < 32 * vec_per_row; idx += 256) {
        const int j = idx / vec_per_row, cv = idx % vec_per_row;
        const int t = t_base + slab * 32 + j;
        const uint4 vv = t < S ? *(const uint4*)(Vg + (size_t)t * DHHV + cv * 8) : make_uint4(0, 0, 0, 0);
        *(uint4*)(Ts + j * VS + cv * 8) = vv;
      }
      __syncthreads();
      if (ni == 0 && slab >= 2) continue;  // positions < 64 never see keys >= 64
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
  __syncthreads();  // Q tile no longer needed: its region becomes the output staging tile

  // ---- epilogue: normalise, round, transpose through LDS, coalesced store
  uint16_t* Hs = Qs;
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int t = 64 * ni + 32 * nb + r;
    const float iv = inv[t];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int w0 = m_wave + 32 * mb + 8 * g4 + 4 * h;
        *(uint2*)(Hs + t * HS + w0) =
            make_uint2(pack_bf16x2(acc[mb][nb][4 * g4 + 0] * iv, acc[mb][nb][4 * g4 + 1] * iv),
                       pack_bf16x2(acc[mb][nb][4 * g4 + 2] * iv, acc[mb][nb][4 * g4 + 3] * iv));
      }
  }
  __syncthreads();
  {
    uint16_t* Hg = a.H + (size_t)bh * S * DHHV + w_tile;
    constexpr int vec_per_row = WT / 8;
    for (int idx = tid; idx < 128 * vec_per_row; idx += 256) {
      const int j = idx / vec_per_row, cv = idx % vec_per_row;
      const int t = t_base + j;
      if (t < S) *(uint4*)(Hg + (size_t)t * DHHV + cv * 8) = *(const uint4*)(Hs + j * HS + cv * 8);
    }
  }
}

template <int WT>
static const char* launch_par_fw_t(const ParFwArgs& a, int BH, hipStream_t stream) {
  const int QS = a.DHQK + 8, HS = WT + 8;
  const size_t q_region = (size_t)128 * (QS > HS ? QS : HS);
  const size_t t_region = (128 * 72 > 32 * (WT + 16)) ? 128 * 72 : 32 * (WT + 16);
  const size_t smem = (q_region + 128 * 136 + t_region) * 2 + (size_t)(6 * 128 + a.DHQK) * 4;
  if (smem > 160 * 1024) return "par_fw: DHQK too large for the LDS-resident Q tile";
  if (hipFuncSetAttribute((const void*)par_fw_kernel<WT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) !=
      hipSuccess)
    return "par_fw: cannot raise the dynamic LDS limit";
  dim3 grid(a.DHHV / WT, a.NC, BH);
  hipLaunchKernelGGL((par_fw_kernel<WT>), grid, dim3(256), smem, stream, a);
  return nullptr;
}

const char* launch_par_fw(const ParFwArgs& a, int BH, hipStream_t stream) {
  if (a.DHQK % 64 != 0 || a.DHHV % 64 != 0) return "par_fw: DHQK and DHHV must be multiples of 64";
  if (a.DHHV % 256 == 0) return launch_par_fw_t<256>(a, BH, stream);
  if (a.DHHV % 128 == 0) return launch_par_fw_t<128>(a, BH, stream);
  return launch_par_fw_t<64>(a, BH, stream);
}

}  // namespace mlstm
