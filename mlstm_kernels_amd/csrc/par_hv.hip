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
//     prefetched several contraction steps ahead in registers,
//   * the 64 rows of Xn this workgroup owns stay resident in LDS (they feed the score matrix, the inter-chunk
//     product and, forward, q.n),
//   * colscale multiplies the fp32 accumulator after the inter-chunk product (positions are accumulator
//     columns), so Xn is never rescaled or re-rounded,
//   * the gated score matrix P is produced cooperatively (fp32 gating, bf16 into LDS); only the blocks on or
//     below the causal diagonal are computed,
//   * Xw^T fragments come from row-major slabs through the transposing LDS read; every slab is fetched from
//     global memory into registers while the previous one is being multiplied.
// A workgroup owns 64 positions (half a chunk).  The resident rows, the gated score matrix and (forward) the
// denominators are built once; then the workgroup walks the value dimension in tiles of WT columns, its WT/MW waves
// splitting a tile.  The footprint (about 73 KB of LDS) lets two workgroups share a CU; at WT = 256, MW = 32 that is
// sixteen waves per CU, four instruction streams per SIMD to overlap memory, LDS and matrix latencies.
//
// Measured on MI355X at B=4, S=16384, 256/512 and not kept: the whole tile's state fragments in flight (PD = 16: spills
// at 128 registers, 0.74 ms against 0.62 ms); four waves of 64 columns (0.61 against 0.585 ms); launching the chunks
// whose states the scan wrote last first, chunk-major (no change: the memory-side cache does not hold them).
#include "common.h"
#include "kernels.h"

namespace mlstm {

#ifndef MLSTM_PAR_HV_MW256
#define MLSTM_PAR_HV_MW256 32
#endif

// PD = how many contraction steps ahead the state fragments are fetched (must divide DHQK / 16).
// MW = value columns per wave (64 or 32): WT / MW waves share the tile.
#define PAR_HV_WPE(WT_, MW_) ((WT_) / (MW_) >= 8 ? 4 : ((WT_) >= 128 ? 2 : 1))
template <int WT, bool IS_DV, int PD, int MW>
__device__ __forceinline__ void par_hv_body(const ParHvArgs& a, const BlockId blk) {
  constexpr int NWAVE = WT / MW;   // each wave owns MW value columns = MB MFMA row blocks
  constexpr int MB = MW / 32;
  constexpr int NTH = 64 * NWAVE;
  constexpr int PS = 128 + 8;      // score matrix row stride: P stored as Ps[n][o]
  constexpr int KS = 64 + 8;       // slab row stride of the streamed score operand
  constexpr int VS = WT + 32;      // slab row stride of the streamed value-side operand (rows 64 bytes apart in the banks)
  constexpr int HS = WT + 8;       // output staging row stride
  const int DHQK = a.DHQK, DHHV = a.DHHV, S = a.S, NC = a.NC;
  const int QS = DHQK + 8;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  const int n_region = 64 * QS;
  uint16_t* Ns = (uint16_t*)smem_raw;  // resident Xn rows [64][DHQK] in fragment order
  uint16_t* Ps = Ns + n_region;
  uint16_t* Ts = Ps + 64 * PS;
  constexpr int t_region = (128 * KS > 32 * VS) ? 128 * KS : 32 * VS;
  float* uu = (float*)(Ts + t_region);  // [128] u_t of the chunk
  float* ww = uu + 128;                 // [128] w_j of the chunk
  float* cs = ww + 128;                 // [64] column scale of this workgroup's positions
  float* inv = cs + 64;                 // forward: [64] 1/(nmax + eps); dV: [128] rho_t of the chunk
  float* rows = inv + 128;              // [8][32] partial row sums of Sbar per score unit (forward)
  float* nperm = rows + 8 * 32;         // [DHQK] n_prev in fragment order (forward)
  float* mcs = nperm + DHQK;            // [64] combined stabiliser of this workgroup's positions (forward)

  // the wave index is made scalar so that branches on it are scalar branches (accumulators stay in place)
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, h = lane >> 5;
#ifdef MLSTM_PAR_TIMING
  unsigned long long tph[7] = {0, 0, 0, 0, 0, 0, 0}, tlast = __builtin_amdgcn_s_memtime();
#define MLSTM_PTICK(p_) { const unsigned long long now_ = __builtin_amdgcn_s_memtime(); tph[p_] += now_ - tlast; tlast = now_; }
#else
#define MLSTM_PTICK(p_)
#endif
  const int bh = blk.z, c = blk.y;
  const int nh = blk.x;                // which half of the chunk's positions
  const int NWT = DHHV / WT;           // column tiles, handled one after the other by this workgroup
  const size_t Sp = (size_t)NC * kChunk;
  const size_t gofs = bh * Sp + (size_t)c * kChunk;
  const int t_base = c * kChunk;
  const int n0 = 64 * nh;              // first position (inside the chunk) of this workgroup
  // live 32-row blocks of the other position index o: forward o = j <= t, dV o = t >= j
  const int ob_lo = IS_DV ? 2 * nh : 0, ob_hi = IS_DV ? 4 : 2 * (nh + 1);
  const uint16_t* Xn_g = (IS_DV ? a.K : a.Q) + (size_t)bh * S * DHQK;
  const uint16_t* Xo_g = (IS_DV ? a.Q : a.K) + (size_t)bh * S * DHQK;
  const uint16_t* Xw_g = (IS_DV ? a.dH : a.V) + (size_t)bh * S * DHHV;

  // ---- phase 0: resident rows, gate vectors (and n_prev) into LDS; first score slab into registers
  constexpr int KV = 128 * 8 / NTH;  // 16-byte vectors per thread per score slab (128 rows x 64 columns)
  uint4 kreg[KV];
  auto load_kslab = [&](int slab) {
#pragma unroll
    for (int v = 0; v < KV; ++v) {
      const int idx = tid + v * NTH;
      const int j = idx >> 3, cv = idx & 7;
      const int t = t_base + j;
      const bool live = j >= 32 * ob_lo && j < 32 * ob_hi && t < S;
      kreg[v] = live ? *(const uint4*)(Xo_g + (size_t)t * DHQK + slab * 64 + cv * 8) : make_uint4(0, 0, 0, 0);
    }
  };
  load_kslab(0);
  // state fragments of the first contraction steps of the first column tile: requested up front, together with
  // everything else this workgroup needs first, so that all of it costs ONE trip to memory (they are consumed in
  // the main phase, after the score phase)
  const int m_wave = wave * MW;  // first value column of this wave inside a column tile
  const int ND = DHQK / 16;
  const uint4* const st_chunk = (const uint4*)a.states + ((size_t)bh * NC + c) * (size_t)(DHHV / 32) * ND * 64 + lane;
  Frag ring[PD][MB];
#define MLSTM_LOAD_RING(wt_, stride_)                                                                      \
  {                                                                                                        \
    const uint4* s0_ = st_chunk + ((size_t)((wt_) * WT + m_wave) / 32 * ND) * 64;                          \
    _Pragma("unroll") for (int p = 0; p < PD; ++p)                                                         \
      _Pragma("unroll") for (int mb = 0; mb < MB; ++mb)                                                    \
        ring[p][mb].u = s0_[(size_t)(mb * ND + p) * (stride_)];                                            \
  }
  MLSTM_LOAD_RING(0, 64)
  {
    // resident rows: all loads of a batch are issued before the first LDS store (a load-store-load-store loop
    // would pay the memory latency once per iteration)
    const int vec_per_row = DHQK / 8;
    constexpr int QB = NTH >= 512 ? 4 : 8;
    for (int base = 0; base < 64 * vec_per_row; base += QB * NTH) {
      u32x4 qrow[QB];
#pragma unroll
      for (int u = 0; u < QB; ++u) {
        const int idx = base + tid + u * NTH;
        const int j = idx / vec_per_row, cv = idx % vec_per_row;
        const int t = t_base + n0 + j;
        const u32x4 z = {0u, 0u, 0u, 0u};
        qrow[u] = (idx < 64 * vec_per_row && t < S) ? *(const u32x4*)(Xn_g + (size_t)t * DHQK + cv * 8) : z;
      }
#pragma unroll
      for (int u = 0; u < QB; ++u) {
        const int idx = base + tid + u * NTH;
        const int j = idx / vec_per_row, cv = idx % vec_per_row;
        if (idx < 64 * vec_per_row) store_perm16(Ns + j * QS, cv, make_uint4(qrow[u][0], qrow[u][1], qrow[u][2], qrow[u][3]));
      }
    }
    for (int idx = tid; idx < 128; idx += NTH) {
      uu[idx] = a.g.u[gofs + idx];
      ww[idx] = a.g.w[gofs + idx];
      if (IS_DV) inv[idx] = a.use_nrow ? 1.f / (a.nrow[gofs + idx] + a.eps) : 1.f;
    }
    for (int idx = tid; idx < 64; idx += NTH)
      cs[idx] = IS_DV ? a.g.abar[gofs + n0 + idx] : a.g.bbar[gofs + n0 + idx] * a.qk_scale;
    if (!IS_DV) {
      for (int d = tid; d < DHQK; d += NTH) nperm[perm16(d)] = a.nstates[((size_t)bh * NC + c) * DHQK + d];
      // fetched with everything else: read from global memory in the denominator phase, the stabiliser costs that
      // phase a whole trip to memory
      for (int idx = tid; idx < 64; idx += NTH) mcs[idx] = a.g.mcomb[gofs + n0 + idx];
    }
  }

  MLSTM_PTICK(0)
  // ---- phase S: score units (32 o x 32 n; unit u = block ob_lo + u/2, position block u%2), dealt round-robin to the
  // waves; contraction over DHQK in slabs of 64
  constexpr int UW = 8 / NWAVE;  // score units per wave
  f32x16 sacc[UW];
#pragma unroll
  for (int k = 0; k < UW; ++k)
#pragma unroll
    for (int i = 0; i < 16; ++i) sacc[k][i] = 0.f;
  const int nslab = DHQK / 64;
  for (int slab = 0; slab < nslab; ++slab) {
    __syncthreads();  // previous slab fully consumed (and phase-0 writes visible on the first pass)
#pragma unroll
    for (int v = 0; v < KV; ++v) {
      const int idx = tid + v * NTH;
      store_perm16(Ts + (idx >> 3) * KS, idx & 7, kreg[v]);
    }
    __syncthreads();
    if (slab + 1 < nslab) load_kslab(slab + 1);
#pragma unroll
    for (int k = 0; k < UW; ++k) {
      // unconditional on purpose: a wave whose block lies above the diagonal multiplies zero rows (its result is
      // dropped at the gating step); a branch here would make the compiler shuttle the score accumulators between
      // the two register files on every iteration
      const int u = wave + k * NWAVE;
      const int ob = ob_lo + (u >> 1), nb = u & 1;
      const int obc = ob < 4 ? ob : 3;
#pragma unroll
      for (int ds = 0; ds < 4; ++ds) {
        Frag A, B;
        A.u = *(const uint4*)(Ts + (32 * obc + r) * KS + 16 * ds + 8 * h);
        B.u = *(const uint4*)(Ns + (32 * nb + r) * QS + slab * 64 + 16 * ds + 8 * h);
        mfma32(sacc[k], A, B);
      }
    }
  }
  MLSTM_PTICK(1)
  // first value slab into registers while the score matrix is gated
  constexpr int VV = 32 * (WT / 8) / NTH;  // 16-byte vectors per thread per value slab (32 rows x WT columns)
  uint4 vreg[VV];
  auto load_vslab = [&](int wt, int ob) {
#pragma unroll
    for (int v = 0; v < VV; ++v) {
      const int idx = tid + v * NTH;
      const int j = idx / (WT / 8), cv = idx % (WT / 8);
      const int t = t_base + 32 * ob + j;
      vreg[v] = t < S ? *(const uint4*)(Xw_g + (size_t)t * DHHV + wt * WT + cv * 8) : make_uint4(0, 0, 0, 0);
    }
  };
  load_vslab(0, ob_lo);
  // gate, mask, round, and write P as Ps[n][o]; forward also accumulates fp32 row sums over j
#pragma unroll
  for (int k = 0; k < UW; ++k) {
    const int u = wave + k * NWAVE;
    const int ob = ob_lo + (u >> 1), nb = u & 1;
    float rsum = 0.f;
    if (ob < ob_hi) {
      const int nl = 32 * nb + r;    // position inside this workgroup's half
      const int n = n0 + nl;         // position inside the chunk
      const float un = IS_DV ? ww[n] : uu[n];  // dV: n is the key position j -> w_j ; forward: n = t -> u_t
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int o0 = 32 * ob + 8 * g4 + 4 * h;
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
          const float val = sacc[k][4 * g4 + e] * a.qk_scale * __expf(ex) * rho[e];
          pv[e] = keep ? val : 0.f;
          rsum += pv[e];
        }
        *(uint2*)(Ps + nl * PS + o0) = make_uint2(pack_bf16x2(pv[0], pv[1]), pack_bf16x2(pv[2], pv[3]));
      }
    }
    if (!IS_DV) {
      const float tot = rsum + __shfl_xor(rsum, 32);
      if (h == 0) rows[u * 32 + r] = tot;  // units above the diagonal publish zero
    }
  }
  __syncthreads();

  MLSTM_PTICK(2)
  // ---- phase D (forward): denominators; NTH/64 threads share a row
  if (!IS_DV) {
    constexpr int TPR = NTH / 64;  // threads per row: 8, 4, 2 or 1
    const int t = tid / TPR, part = tid % TPR;
    const int seg = DHQK / TPR;
    const uint16_t* qrow = Ns + t * QS + part * seg;
    const float* np = nperm + part * seg;
    float dot = 0.f;
    for (int d = 0; d < seg; d += 8) {
      const uint4 qv = *(const uint4*)(qrow + d);
      const uint32_t qq[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        dot += __uint_as_float(qq[p] << 16) * np[d + 2 * p];
        dot += __uint_as_float(qq[p] & 0xffff0000u) * np[d + 2 * p + 1];
      }
    }
#pragma unroll
    for (int o = TPR / 2; o > 0; o >>= 1) dot += __shfl_xor(dot, o);
    if (part == 0) {
      float nmax = 1.f, iv = 1.f;
      if (a.use_nrow) {
        float den = cs[t] * dot;
#pragma unroll
        for (int ob4 = 0; ob4 < 4; ++ob4) den += rows[(2 * ob4 + (t >> 5)) * 32 + (t & 31)];
        const float mc = mcs[t];
        const float floor_v = a.sig_gate ? 1.f : __expf(-mc);
        nmax = fmaxf(fabsf(den), floor_v);
        iv = 1.f / (nmax + a.eps);
      }
      inv[t] = iv;
      {
        a.nrow_out[gofs + n0 + t] = nmax;
        const int tg = t_base + n0 + t;
        if (tg < S) {
          if (a.n_out != nullptr) a.n_out[(size_t)bh * S + tg] = nmax;
          if (a.m_out != nullptr) a.m_out[(size_t)bh * S + tg] = mcs[t];
        }
      }
    }
  }

  MLSTM_PTICK(3)
  // ---- main phase, once per column tile: Out^T = (State^T Xn^T) * colscale + Xw^T P.  The resident rows, the gated
  // score matrix and the denominators above are shared by all column tiles of this (chunk, position half).
  const int q16 = (lane >> 4) & 1, i16 = lane & 15;
  const int krow = 8 * h + (i16 >> 2), ncol = 16 * q16 + 4 * (i16 & 3);
  for (int wt = 0; wt < NWT; ++wt) {
    f32x16 acc[MB][2];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.f;
    {
      const uint4* s0 = st_chunk + ((size_t)(wt * WT + m_wave) / 32 * ND) * 64;
      for (int ds0 = 0; ds0 < ND; ds0 += PD) {
#pragma unroll
        for (int p = 0; p < PD; ++p) {
          const int ds = ds0 + p;
          Frag A[MB], B[2];
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) A[mb] = ring[p][mb];
          if (ds + PD < ND) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) ring[p][mb].u = s0[(size_t)(mb * ND + ds + PD) * 64];
          }
#pragma unroll
          for (int nb = 0; nb < 2; ++nb) B[nb].u = *(const uint4*)(Ns + (32 * nb + r) * QS + 16 * ds + 8 * h);
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) mfma32(acc[mb][nb], A[mb], B[nb]);
        }
      }
    }
    // the next column tile's first state fragments travel while this tile finishes.  The load is unconditional (a
    // conditional one makes the compiler spill ring registers); after the last tile every ring slot re-requests one
    // and the same fragment (stride 0), which costs a cache hit instead of 64 KB of fetches from HBM.
    {
      const bool more_tiles = wt + 1 < NWT;
      const int wt_next = more_tiles ? wt + 1 : wt;
      const int ring_stride = more_tiles ? 64 : 0;
      MLSTM_LOAD_RING(wt_next, ring_stride)
    }
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      const float sc = cs[32 * nb + r];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) acc[mb][nb] *= sc;
    }
    MLSTM_PTICK(4)
    for (int ob = ob_lo; ob < ob_hi; ++ob) {
      __syncthreads();  // slab buffer free (first pass: P / inv written, score slabs consumed; later: staging stored)
#pragma unroll
      for (int v = 0; v < VV; ++v) {
        const int idx = tid + v * NTH;
        *(uint4*)(Ts + (idx / (WT / 8)) * VS + (idx % (WT / 8)) * 8) = vreg[v];
      }
      __syncthreads();
      {
        // next slab of this tile, or the first slab of the next tile (the very last one re-requests itself)
        const bool more = ob + 1 < ob_hi;
        const int wt_n = more ? wt : (wt + 1 < NWT ? wt + 1 : wt);
        load_vslab(wt_n, more ? ob + 1 : ob_lo);
      }
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
        for (int nb = 0; nb < 2; ++nb) B[nb].u = *(const uint4*)(Ps + (32 * nb + r) * PS + 32 * ob + 16 * jl + 8 * h);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
          for (int nb = 0; nb < 2; ++nb) mfma32(acc[mb][nb], A[mb], B[nb]);
      }
    }
    MLSTM_PTICK(5)

    // ---- epilogue: (normalise,) round, transpose through the slab buffer (32 positions at a time), coalesced store
    uint16_t* Og = a.Out + (size_t)bh * S * DHHV + wt * WT;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      __syncthreads();  // slab buffer free (last value slab consumed / previous half stored)
      const float iv = IS_DV ? 1.f : inv[32 * nb + r];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int w0 = m_wave + 32 * mb + 8 * g4 + 4 * h;
          *(uint2*)(Ts + r * HS + w0) =
              make_uint2(pack_bf16x2(acc[mb][nb][4 * g4 + 0] * iv, acc[mb][nb][4 * g4 + 1] * iv),
                         pack_bf16x2(acc[mb][nb][4 * g4 + 2] * iv, acc[mb][nb][4 * g4 + 3] * iv));
        }
      __syncthreads();
      constexpr int vec_per_row = WT / 8;
      for (int idx = tid; idx < 32 * vec_per_row; idx += NTH) {
        const int j = idx / vec_per_row, cv = idx % vec_per_row;
        const int t = t_base + n0 + 32 * nb + j;
        // non-temporal: nobody in this launch reads the output, it should not evict shared operands from the L2
        if (t < S) __builtin_nontemporal_store(*(const u32x4*)(Ts + j * HS + cv * 8), (u32x4*)(Og + (size_t)t * DHHV + cv * 8));
      }
    }
  }
#undef MLSTM_LOAD_RING
  MLSTM_PTICK(6)
#ifdef MLSTM_PAR_TIMING
  if (blk.y == a.NC / 2 && blk.z == 0 && lane == 0)
    for (int p = 0; p < 7; ++p) a.timing[(blk.x * 4 + (wave & 3)) * 8 + p] = tph[p];
#endif
}

template <int WT, bool IS_DV, int PD, int MW>
__global__ __launch_bounds__(64 * (WT / MW))
    __attribute__((amdgpu_waves_per_eu(PAR_HV_WPE(WT, MW), PAR_HV_WPE(WT, MW)))) void par_hv_kernel(ParHvArgs a) {
  par_hv_body<WT, IS_DV, PD, MW>(a, xcd_block_id());  // both halves of a chunk share operands: same XCD
}

template <int WT, bool IS_DV, int PD, int MW>
static const char* launch_par_hv_pd(const ParHvArgs& a, int BH, hipStream_t stream) {
  const int QS = a.DHQK + 8;
  const size_t n_region = (size_t)64 * QS;
  const size_t t_region = (128 * 72 > 32 * (WT + 32)) ? 128 * 72 : 32 * (WT + 32);
  const size_t smem = (n_region + 64 * 136 + t_region) * 2 + (size_t)(128 * 3 + 64 + 8 * 32 + a.DHQK + 64) * 4;
  if (smem > 160 * 1024) return "par_hv: DHQK too large for the LDS-resident tile";
  if (hipFuncSetAttribute((const void*)par_hv_kernel<WT, IS_DV, PD, MW>, hipFuncAttributeMaxDynamicSharedMemorySize,
                          (int)smem) != hipSuccess)
    return "par_hv: cannot raise the dynamic LDS limit";
  dim3 grid(2, a.NC, BH);
  hipLaunchKernelGGL((par_hv_kernel<WT, IS_DV, PD, MW>), grid, dim3(64 * (WT / MW)), smem, stream, a);
  return nullptr;
}

template <int WT, bool IS_DV>
static const char* launch_par_hv_t(const ParHvArgs& a, int BH, hipStream_t stream) {
  // eight steps ahead (64 registers of fragments in flight per lane) measured 8 % faster than four at 256/512
  constexpr int MW = WT == 256 ? MLSTM_PAR_HV_MW256 : 64;
  if (a.DHQK % 128 == 0) return launch_par_hv_pd<WT, IS_DV, 8, MW>(a, BH, stream);
  return launch_par_hv_pd<WT, IS_DV, 4, MW>(a, BH, stream);
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
