// Chunk-parallel kernels whose output tile spans value columns: the forward output H and the gradient dV.
//
// forward (mlstm_kernels/torch/chunkwise/native/fw.py:171-212 in the reference), per chunk:
//   Sbar[t][j] = (q_t . k_j)/sqrt(DHQK) * exp(u_t - w_j)   (j <= t)
//   H[t][:]    = ( bbar_t/sqrt(DHQK) * q_t^T C_prev + sum_j Sbar[t][j] v_j ) / (max(|den_t|, floor_t) + eps)
//   den_t      = bbar_t/sqrt(DHQK) * q_t . n_prev + sum_j Sbar[t][j]
// backward dV (mlstm_kernels/torch/chunkwise/native/bw.py:153-198), per chunk:
//   dV[j][:]   = sum_t Sbar[t][j] rho_t dH[t][:]  +  abar_j * k_j^T dC_next          rho_t = 1/(nrow_t + eps)
//
// Chunk states are kept only every `stride`-th chunk (the counterpart of the reference's chunk_size_inter <
// chunk_size_intra with save_states_every_nth_chunk, mlstm_kernels/triton/chunkwise/kernel_param_heuristics.py:28-31,
// 118-121).  A chunk c whose own boundary state was not kept uses the nearest kept one and adds the chunks in between
// as further score blocks without a causal mask: with c0 the last kept boundary at or before c,
//   H[t]  = bbar_t e^{G(c0,c) + m_{c0} - m_c}/sqrt(d) q_t^T C_{c0}  +  sum_{c'=c0}^{c} sum_{j in c'} Sbar'[t][j] v_j,
//   Sbar'[t][j] = (q_t . k_j)/sqrt(d) exp(u_t - w_j + G(c',c)),   G(a,b) = sum_{x=a}^{b-1} (sum of logsig(f) over chunk x)
// (u, w are the within-chunk gate vectors of the chunk t resp. j lives in; every exponent stays <= 0), and dV is the
// mirror image with the nearest kept dC boundary at or after the chunk.  The denominators need no change: n is
// kept for every chunk (it is a vector).
//
// Both are the same GEMM chain on a transposed output tile  Out^T[w][n]  (value columns x chunk positions):
//   Out^T = ( State^T[w][d] . Xn^T[d][n] ) * colscale[n]  +  sum over source chunks  Xw^T[w][o] . P[o][n]
// with  n = query position t, o = key position j, Xn = Q, Xw = V, State = C       (forward)
//       n = key position j,   o = query position t, Xn = K, Xw = dH, State = dC   (dV)
//   * State^T arrives as ready-made bf16 MFMA fragments written by the scan kernel (16 B per lane, no LDS),
//     prefetched several contraction steps ahead in registers,
//   * the 64 rows of Xn this workgroup owns stay resident in LDS (they feed the score blocks, the inter-chunk
//     product and, forward, q.n),
//   * colscale multiplies the fp32 accumulator after the inter-chunk product (positions are accumulator
//     columns), so Xn is never rescaled or re-rounded,
//   * per source chunk the gated score block P (64 x 128) is produced cooperatively (fp32 gating, bf16 into LDS)
//     and consumed at once by all value columns of the group: the accumulators of up to two column tiles are live
//     together, so a score block is computed once and never kept,
//   * Xw^T fragments come from row-major slabs through the transposing LDS read; every slab is fetched from
//     global memory into registers while the previous one is being multiplied.
// A workgroup owns 64 positions (half a chunk) and walks the value dimension in groups of NTG tiles of WT columns, its
// WT/MW waves splitting a tile.  The footprint (about 73 KB of LDS) lets two workgroups share a CU; at WT = 256,
// MW = 32 that is sixteen waves per CU, four instruction streams per SIMD to overlap memory, LDS and matrix latencies.
#include "common.h"
#include "kernels.h"

namespace mlstm {

// PD = how many contraction steps ahead the state fragments are fetched (must divide DHQK / 16).
// MW = value columns per wave (64 or 32): WT / MW waves share a tile.  NTG = column tiles per group (1 or 2).
#define PAR_HV_WPE(WT_, MW_) ((WT_) / (MW_) >= 8 ? 4 : ((WT_) >= 128 ? 2 : 1))
template <int WT, int NTG, bool IS_DV, int PD, int MW, bool HEAD_NORM, bool F16>
__device__ __forceinline__ void par_hv_body(const ParHvArgs& a, const BlockId blk) {
  constexpr int NWAVE = WT / MW;   // each wave owns MW value columns of every tile of the group = MB MFMA row blocks
  constexpr int MB = MW / 32;
  constexpr int NTH = 64 * NWAVE;
  constexpr int GW = WT * NTG;     // value columns per group
  constexpr int VR = 8192 / GW;    // rows per value slab: a slab is 16 KB, like a score slab
  constexpr int PS = 128 + 8;      // score block row stride: P stored as Ps[n][o]
  constexpr int KS = 64 + 8;       // slab row stride of the streamed score operand
  constexpr int VS = GW + 32;      // slab row stride of the streamed value-side operand (rows 64 bytes apart in the banks)
  constexpr int HS = WT + 8;       // output staging row stride
  const int DHQK = a.DHQK, DHHV = a.DHHV, S = a.S, NC = a.NC;
  const int QS = DHQK + 8;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  const int n_region = 64 * QS;
  uint16_t* Ns = (uint16_t*)smem_raw;  // resident Xn rows [64][DHQK] in fragment order
  uint16_t* Ps = Ns + n_region;
  uint16_t* Ts = Ps + 64 * PS;
  constexpr int t_region = (128 * KS > VR * VS) ? 128 * KS : VR * VS;
  static_assert(VR >= 16 && VR <= 128, "value slabs hold 16 to 128 rows");
  float* nvec = (float*)(Ts + t_region);  // [64] gate vector of this workgroup's positions: u_t (forward) / w_j (dV)
  float* ovec = nvec + 64;              // [128] gate vector of the source chunk: w_j (forward) / u_t (dV)
  float* orho = ovec + 128;             // [128] dV: rho_t of the source chunk
  float* cs = orho + 128;               // [64] column scale of the inter-chunk product
  float* inv = cs + 64;                 // [64] forward: 1/(nmax + eps)
  float* rows = inv + 64;               // [8][32] partial row sums of Sbar per score unit (forward)
  float* nperm = rows + 8 * 32;         // [DHQK] n_prev in fragment order (forward)
  float* mcs = nperm + DHQK;            // [64] combined stabiliser of this workgroup's positions (forward)
  float* cs0 = mcs + 64;                // [64] forward: bbar_t/sqrt(d), the weight of q.n_prev in the denominator

  // the wave index is made scalar so that branches on it are scalar branches (accumulators stay in place)
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, h = lane >> 5;
  const int bh = blk.z, c = blk.y;
  const int nh = blk.x;                // which half of the chunk's positions
  const int NG = DHHV / GW;            // column groups, handled one after the other by this workgroup
  const size_t Sp = (size_t)NC * kChunk;
  const size_t hofs = bh * Sp;
  const size_t gofs = hofs + (size_t)c * kChunk;
  const int t_base = c * kChunk;
  const int n0 = 64 * nh;              // first position (inside the chunk) of this workgroup
  const int stride = a.stride;
  const int slot = c / stride;         // kept boundary state this chunk uses
  // source chunks of the score blocks: forward c0 .. c, dV c .. c1.  They are walked with the own chunk LAST (forward
  // upwards, dV downwards): a far chunk's rows are then requested when this workgroup starts, which is when the
  // workgroups of that chunk -- neighbours in launch order on the same XCD -- request them as their own, so the two
  // meet in the L2 (walked the other way round, dV fetched 47 % more bytes than it needs).
  const int sc_lo = IS_DV ? c : slot * stride;
  const int sc_hi = IS_DV ? min(slot * stride + stride - 1, NC - 1) : c;
  const int sc_first = IS_DV ? sc_hi : sc_lo, sc_step = IS_DV ? -1 : 1;
  const uint16_t* Xn_g = (IS_DV ? a.K : a.Q) + (size_t)bh * S * DHQK;
  const uint16_t* Xo_g = (IS_DV ? a.Q : a.K) + (size_t)bh * S * DHQK;
  const uint16_t* Xw_g = (IS_DV ? a.dH : a.V) + (size_t)bh * S * DHHV;
  const float* graw = a.g.graw + (size_t)bh * NC;
  const float* mst = a.g.mstates + (size_t)bh * (NC + 1);

  // live 32-row blocks of the other position index o inside source chunk sc: own chunk forward o = j <= t, dV
  // o = t >= j; any other source chunk is live as a whole
  auto ob_range = [&](int sc, int& lo, int& hi) {
    lo = (IS_DV && sc == c) ? 2 * nh : 0;
    hi = (!IS_DV && sc == c) ? 2 * (nh + 1) : 4;
  };

  // ---- streamed operands.  The score operand (Xo rows, 64 head-dim columns per slab) and the value-side operand (Xw
  // rows, GW columns per slab) of all source chunks form ONE sequence of steps: per source chunk DHQK/64 score slabs,
  // then the value slabs that cover its live rows.  Every slab is 16 KB (SV 16-byte vectors per thread), so the same
  // two register sets serve both kinds, and the slab of step s+2 is requested while step s is being multiplied: a
  // workgroup always has two slabs on their way, whatever phase it is in.  (With one slab in flight a step cannot be
  // shorter than a trip to the L2, several times its LDS and matrix work.)
  constexpr int SV = 128 * 8 / NTH;      // 16-byte vectors per thread per slab
  constexpr int VRP = NTH / (GW / 8);    // value-slab rows covered by one sweep of the workgroup
  static_assert(SV * VRP == VR, "a value slab is as large as a score slab");
  constexpr int OVN = NTH >= 128 ? 1 : 128 / NTH;  // gate-vector entries per thread (a workgroup may be one wave)
  uint4 sA[SV], sB[SV];
  float ovA[OVN], orA[OVN], ovB[OVN], orB[OVN];
  // Streamed rows are addressed as a uniform base plus a 32-bit byte offset per lane (offsets inside one (batch, head)
  // fit 32 bits, checked by the launcher), which keeps the addresses out of the vector registers.  Rows past the end
  // of the sequence are read from its last row instead of being zeroed: their gate factor is zero (forward) or the
  // value rows they meet are stored as zeros (dV), and rows of dead blocks only feed score units nobody reads.
  const char* const Xo_b = (const char*)Xo_g;
  const char* const Xw_b = (const char*)Xw_g;
  const int nslab = DHQK / 64;
  // live value slabs of source chunk sc: [sl_lo, sl_hi)
  auto vslab_range = [&](int sc, int& sl_lo, int& sl_hi) {
    int lo, hi;
    ob_range(sc, lo, hi);
    sl_lo = 32 * lo / VR;
    sl_hi = (32 * hi + VR - 1) / VR;
  };
  // The two register sets alternate step by step; so that the set of a step is known at compile time, each phase
  // (score slabs of a source chunk, value slabs of a source chunk) is padded to an even number of steps -- a padding
  // step moves nothing and multiplies nothing.  MAYPAD is false for the shapes whose phases are even anyway.
  constexpr bool MAYPAD_V = VR > 32;  // value phases of 64 or 128 rows per slab can be a single slab
  const bool maypad_k = (nslab & 1) != 0;
  const int nk2 = nslab + (nslab & 1);
  struct Target {
    int sc, kind, idx;  // kind 0: score slab idx; kind 1: value slab idx (absolute slab index inside the chunk)
    bool real;
  };
  // the step two positions after (sc, kind, rel) in the padded sequence (rel = position inside its phase)
  auto ahead2 = [&](int sc, int kind, int rel) {
    int sl_lo, sl_hi;
    vslab_range(sc, sl_lo, sl_hi);
    const int nv = sl_hi - sl_lo, nv2 = nv + (nv & 1);
    Target t;
    int r2 = rel + 2;
    if (kind == 0) {
      if (r2 < nk2) {
        t = {sc, 0, r2, r2 < nslab};
      } else {
        r2 -= nk2;
        t = {sc, 1, sl_lo + r2, r2 < nv};
      }
    } else {
      if (r2 < nv2) {
        t = {sc, 1, sl_lo + r2, r2 < nv};
      } else {
        r2 -= nv2;
        t = {sc + sc_step, 0, r2, sc != c && r2 < nslab};  // the own chunk is the last one
      }
    }
    if (!t.real) t = {sc_first, 0, 0, false};
    return t;
  };
  // request a slab (and the gate vectors of its source chunk) into register set R_.  A target that is not real makes
  // every lane request one and the same 16 bytes (a cache hit nobody waits for), so that the registers of the set are
  // defined on every path.
#define MLSTM_LOAD_AT(R_, OV_, OR_, grp_, tg_)                                                                       \
  {                                                                                                                  \
    const Target nx_ = (tg_);                                                                                        \
    const int tl_ = opaque(tid);                                                                                     \
    const bool isv_ = nx_.kind != 0;                                                                                 \
    const uint32_t row0_ = isv_ ? (uint32_t)tl_ / (GW / 8) : (uint32_t)tl_ >> 3;                                     \
    const uint32_t unit_ = nx_.real ? (isv_ ? ((uint32_t)tl_ % (GW / 8)) * 16 : ((uint32_t)tl_ & 7) * 16) : 0u;      \
    const uint32_t rstep_ = isv_ ? VRP : NTH / 8;                                                                    \
    const uint32_t rbase_ = (uint32_t)(nx_.sc * kChunk) + (isv_ ? (uint32_t)(VR * nx_.idx) : 0u);                    \
    const uint32_t pitch_ = isv_ ? (uint32_t)(DHHV * 2) : (uint32_t)(DHQK * 2);                                      \
    const uint32_t coff_ = isv_ ? (uint32_t)((grp_) * GW * 2) : (uint32_t)(nx_.idx * 128);                           \
    const char* const base_ = isv_ ? Xw_b : Xo_b;                                                                    \
    _Pragma("unroll") for (int v = 0; v < SV; ++v) {                                                                 \
      const uint32_t t_ = nx_.real ? min(rbase_ + row0_ + v * rstep_, (uint32_t)(S - 1)) : rbase_;                   \
      R_[v] = *(const uint4*)(base_ + (t_ * pitch_ + coff_ + unit_));                                                \
    }                                                                                                                \
    _Pragma("unroll") for (int e = 0; e < OVN; ++e) {                                                                \
      const int idx_ = min(tl_ + e * NTH, 127);                                                                      \
      OV_[e] = (IS_DV ? a.g.u : a.g.w)[hofs + (size_t)nx_.sc * kChunk + idx_];                                       \
      OR_[e] = (IS_DV && a.use_nrow) ? a.nrow[hofs + (size_t)nx_.sc * kChunk + idx_] : 1.f;                          \
    }                                                                                                                \
  }
  MLSTM_LOAD_AT(sA, ovA, orA, 0, (Target{sc_first, 0, 0, true}))
  MLSTM_LOAD_AT(sB, ovB, orB, 0, (Target{sc_first, 0, nslab > 1 ? 1 : 0, nslab > 1}))
  // state fragments of the first contraction steps of the first column tile: requested up front, together with
  // everything else this workgroup needs first, so that all of it costs ONE trip to memory
  const int m_wave = wave * MW;  // first value column of this wave inside a column tile
  const int ND = DHQK / 16;
  const int NCS = (NC + stride - 1) / stride;
  const char* const st_chunk = (const char*)((const uint4*)a.states + ((size_t)bh * NCS + slot) * (size_t)(DHHV / 32) * ND * 64);
  Frag ring[PD][MB];
  // state fragments of value columns col_ .. col_ + 31 (fragment block col_ / 32), contraction step ds_
#define MLSTM_STATE_FRAG(col_, ds_) \
  (*(const uint4*)(st_chunk + (size_t)(((col_) / 32) * ND + (ds_)) * 1024 + st_lane))
#define MLSTM_LOAD_RING(col0_)                                                                             \
  {                                                                                                        \
    const uint32_t st_lane = opaque(lane) * 16;                                                            \
    _Pragma("unroll") for (int p = 0; p < PD; ++p)                                                         \
      _Pragma("unroll") for (int mb = 0; mb < MB; ++mb)                                                    \
        ring[p][mb].u = MLSTM_STATE_FRAG((col0_) + m_wave + 32 * mb, p);                                   \
  }
  MLSTM_LOAD_RING(0)
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
    if (tid < 64) {
      // weight of the kept boundary state for this chunk: the decay over the chunks between the boundary and this
      // one, re-stabilised (1 when the boundary is the chunk's own)
      float gsum = 0.f, xs;
      if (IS_DV) {
        for (int x = c + 1; x <= sc_hi; ++x) gsum += graw[x];
        xs = sc_hi > c ? __expf(gsum + mst[c + 1] - mst[sc_hi + 1]) : 1.f;
      } else {
        for (int x = sc_lo; x < c; ++x) gsum += graw[x];
        xs = sc_lo < c ? __expf(gsum + mst[sc_lo] - mst[c]) : 1.f;
      }
      const float base = IS_DV ? a.g.abar[gofs + n0 + tid] : a.g.bbar[gofs + n0 + tid] * a.qk_scale;
      cs[tid] = base * xs;
      nvec[tid] = IS_DV ? a.g.w[gofs + n0 + tid] : a.g.u[gofs + n0 + tid];
      if (!IS_DV) {
        cs0[tid] = base;
        // fetched with everything else: read from global memory in the denominator phase, the stabiliser costs that
        // phase a whole trip to memory
        mcs[tid] = a.g.mcomb[gofs + n0 + tid];
      }
    }
    if (!IS_DV) {
      // the scan hands n over as three partial vectors per chunk (their sum carries the full fp32 precision)
      for (int d = tid; d < DHQK; d += NTH) {
        const float* np3 = a.nstates + ((size_t)bh * NC + c) * 3 * DHQK + d;
        nperm[perm16(d)] = (np3[0] + np3[DHQK]) + np3[2 * DHQK];
      }
    }
  }

  constexpr int UW = 8 / NWAVE;  // score units per wave

  // One score-slab step with register set R_: Ts <- Xo rows x 64 head-dim columns of slab ks_; score units (32 o x 32 n;
  // unit u = block ob_lo + u/2, position block u%2) dealt round-robin to the waves.
#define MLSTM_K_STEP(R_, OV_, OR_, ks_)                                                                              \
  {                                                                                                                  \
    const bool valid_ = !maypad_k || (ks_) < nslab;                                                                  \
    if (valid_) {                                                                                                    \
      const int tv = opaque(tid);                                                                                    \
      __syncthreads(); /* previous slab / output staging fully consumed */                                          \
      _Pragma("unroll") for (int v = 0; v < SV; ++v) {                                                               \
        const int idx = tv + v * NTH;                                                                                \
        store_perm16(Ts + (idx >> 3) * KS, idx & 7, R_[v]);                                                          \
      }                                                                                                              \
      if ((ks_) == 0) {                                                                                              \
        _Pragma("unroll") for (int e = 0; e < OVN; ++e) {                                                            \
          const int idx = tv + e * NTH;                                                                              \
          if (idx < 128) {                                                                                           \
            ovec[idx] = OV_[e];                                                                                      \
            if (IS_DV) orho[idx] = a.use_nrow ? 1.f / (OR_[e] + a.eps) : 1.f;                                        \
          }                                                                                                          \
        }                                                                                                            \
      }                                                                                                              \
      __syncthreads();                                                                                               \
    }                                                                                                                \
    MLSTM_LOAD_AT(R_, OV_, OR_, grp, ahead2(sc, 0, (ks_)))                                                           \
    if (valid_) {                                                                                                    \
      const int ln = opaque(lane);                                                                                   \
      const int r = ln & 31, h = ln >> 5;                                                                            \
      _Pragma("unroll") for (int k = 0; k < UW; ++k) {                                                               \
        /* unconditional on purpose: a wave whose block lies above the diagonal multiplies rows nobody reads */    \
        const int u = wave + k * NWAVE;                                                                              \
        const int ob = ob_lo + (u >> 1), nb = u & 1;                                                                 \
        const int obc = ob < 4 ? ob : 3;                                                                             \
        _Pragma("unroll") for (int ds = 0; ds < 4; ++ds) {                                                           \
          Frag A, B;                                                                                                 \
          A.u = *(const uint4*)(Ts + (32 * obc + r) * KS + 16 * ds + 8 * h);                                         \
          B.u = *(const uint4*)(Ns + (32 * nb + r) * QS + (ks_) * 64 + 16 * ds + 8 * h);                             \
          mfma32<F16>(sacc[k], A, B);                                                                                     \
        }                                                                                                            \
      }                                                                                                              \
    }                                                                                                                \
  }
  // One value-slab step with register set R_: Ts <- VR rows of Xw x GW columns (slab sl_lo + vs_ of the chunk);
  // Out^T += Xw^T P over the live 16-row steps of the slab, for every value column of the group.
#define MLSTM_V_STEP(R_, OV_, OR_, vs_)                                                                              \
  {                                                                                                                  \
    const bool valid_ = !MAYPAD_V || (vs_) < nv;                                                                     \
    const int sl_ = sl_lo + (vs_);                                                                                   \
    if (valid_) {                                                                                                    \
      const int tv = opaque(tid);                                                                                    \
      __syncthreads(); /* slab buffer free (first pass: P written, score slabs consumed) */                         \
      _Pragma("unroll") for (int v = 0; v < SV; ++v) {                                                               \
        const int j = tv / (GW / 8) + v * VRP;                                                                       \
        const bool inside = sc * kChunk + VR * sl_ + j < S;                                                          \
        *(uint4*)(Ts + j * VS + (tv % (GW / 8)) * 8) = inside ? R_[v] : make_uint4(0, 0, 0, 0);                      \
      }                                                                                                              \
      __syncthreads();                                                                                               \
    }                                                                                                                \
    MLSTM_LOAD_AT(R_, OV_, OR_, grp, ahead2(sc, 1, (vs_)))                                                           \
    if (valid_) {                                                                                                    \
      const int ln = opaque(lane);                                                                                   \
      const int r = ln & 31, h = ln >> 5;                                                                            \
      const int q16 = (ln >> 4) & 1, i16 = ln & 15;                                                                  \
      const int krow = 8 * h + (i16 >> 2), ncol = 16 * q16 + 4 * (i16 & 3);                                          \
      const int row_lo = max(32 * ob_lo, VR * sl_), row_hi = min(32 * ob_hi, VR * (sl_ + 1));                        \
      for (int row = row_lo; row < row_hi; row += 16) {                                                              \
        const int jl = (row - VR * sl_) >> 4;                                                                        \
        Frag B[2];                                                                                                   \
        _Pragma("unroll") for (int nb = 0; nb < 2; ++nb)                                                             \
          B[nb].u = *(const uint4*)(Ps + (32 * nb + r) * PS + row + 8 * h);                                          \
        _Pragma("unroll") for (int tl = 0; tl < NTG; ++tl) {                                                         \
          Frag A[MB];                                                                                                \
          _Pragma("unroll") for (int mb = 0; mb < MB; ++mb) {                                                        \
            const uint16_t* p = Ts + (16 * jl + krow) * VS + (tl * WT + m_wave + 32 * mb + ncol);                    \
            A[mb].d[0] = lds_read_tr16(p);                                                                           \
            A[mb].d[1] = lds_read_tr16(p + 4 * VS);                                                                  \
          }                                                                                                          \
          _Pragma("unroll") for (int mb = 0; mb < MB; ++mb)                                                          \
            _Pragma("unroll") for (int nb = 0; nb < 2; ++nb) mfma32<F16>(acc[tl][mb][nb], A[mb], B[nb]);                  \
        }                                                                                                            \
      }                                                                                                              \
    }                                                                                                                \
  }

  for (int grp = 0; grp < NG; ++grp) {
    f32x16 acc[NTG][MB][2];
#pragma unroll
    for (int tl = 0; tl < NTG; ++tl)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[tl][mb][nb][i] = 0.f;
    // later groups request their first two slabs only now (the first group's travel since the kernel started)
    if (grp > 0) {
      MLSTM_LOAD_AT(sA, ovA, orA, grp, (Target{sc_first, 0, 0, true}))
      MLSTM_LOAD_AT(sB, ovB, orB, grp, (Target{sc_first, 0, nslab > 1 ? 1 : 0, nslab > 1}))
    }
    __syncthreads();  // phase-0 writes visible (later groups: the previous group's output staging is stored)
    // ---- inter-chunk product, tile by tile: Out^T = State^T Xn^T
#pragma unroll
    for (int tl = 0; tl < NTG; ++tl) {
      const int col0 = grp * GW + tl * WT;
      for (int ds0 = 0; ds0 < ND; ds0 += PD) {
        const int ln = opaque(lane);
        const int r = ln & 31, h = ln >> 5;
        const uint32_t st_lane = ln * 16;
#pragma unroll
        for (int p = 0; p < PD; ++p) {
          const int ds = ds0 + p;
          Frag A[MB], B[2];
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) A[mb] = ring[p][mb];
          {
            // unconditional (the last PD steps re-request the tile's last fragment, a cache hit): a conditional load
            // makes the compiler park ring registers in scratch memory, with a full wait for the load behind it
            const int dn = min(ds + PD, ND - 1);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) ring[p][mb].u = MLSTM_STATE_FRAG(col0 + m_wave + 32 * mb, dn);
          }
#pragma unroll
          for (int nb = 0; nb < 2; ++nb) B[nb].u = *(const uint4*)(Ns + (32 * nb + r) * QS + 16 * ds + 8 * h);
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) mfma32<F16>(acc[tl][mb][nb], A[mb], B[nb]);
        }
      }
      // the next tile's first state fragments travel while this one finishes
      if (tl + 1 < NTG) MLSTM_LOAD_RING(col0 + WT)
    }
    {
      const int r = opaque(lane) & 31;
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        const float sc = cs[32 * nb + r];
#pragma unroll
        for (int tl = 0; tl < NTG; ++tl)
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) acc[tl][mb][nb] *= sc;
      }
    }

    // ---- source chunks: score block, gated into Ps, then Out^T += Xw^T P for every value column of the group
    for (int sc = sc_first; sc >= sc_lo && sc <= sc_hi; sc += sc_step) {
      int ob_lo, ob_hi;
      ob_range(sc, ob_lo, ob_hi);
      int sl_lo, sl_hi;
      vslab_range(sc, sl_lo, sl_hi);
      const int nv = sl_hi - sl_lo;
      const bool own = sc == c;
      f32x16 sacc[UW];
#pragma unroll
      for (int k = 0; k < UW; ++k)
#pragma unroll
        for (int i = 0; i < 16; ++i) sacc[k][i] = 0.f;
      for (int ks = 0; ks < nk2; ks += 2) {
        MLSTM_K_STEP(sA, ovA, orA, ks)
        MLSTM_K_STEP(sB, ovB, orB, ks + 1)
      }
      // gate, mask, round, and write P as Ps[n][o]; forward also accumulates fp32 row sums over j of the own chunk
      {
        // decay between the key chunk and the query chunk of this block (0 for the own chunk)
        float gs = 0.f;
        for (int x = (IS_DV ? c : sc); x < (IS_DV ? sc : c); ++x) gs += graw[x];
        const int lg = opaque(lane);
        const int r = lg & 31, h = lg >> 5;
#pragma unroll
        for (int k = 0; k < UW; ++k) {
          const int u = wave + k * NWAVE;
          const int ob = ob_lo + (u >> 1), nb = u & 1;
          float rsum = 0.f;
          if (ob < ob_hi) {
            const int nl = 32 * nb + r;    // position inside this workgroup's half
            const int n = n0 + nl;         // position inside the chunk
            const float un = nvec[nl] + (IS_DV ? -gs : gs);
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
              const int o0 = 32 * ob + 8 * g4 + 4 * h;
              const float4 xo = *(const float4*)(ovec + o0);
              const float xov[4] = {xo.x, xo.y, xo.z, xo.w};
              float rho[4] = {1.f, 1.f, 1.f, 1.f};
              if (IS_DV) {
                const float4 rr = *(const float4*)(orho + o0);
                rho[0] = rr.x; rho[1] = rr.y; rho[2] = rr.z; rho[3] = rr.w;
              }
              float pv[4];
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                // exponent u_t - w_j (+ the decay between the chunks) and, in the own chunk, the causal mask j <= t
                const float ex = IS_DV ? (xov[e] - un) : (un - xov[e]);
                const bool keep = !own || (IS_DV ? (n <= o0 + e) : (o0 + e <= n));
                const float val = sacc[k][4 * g4 + e] * a.qk_scale * __expf(ex) * rho[e];
                pv[e] = keep ? val : 0.f;
                rsum += pv[e];
              }
              *(uint2*)(Ps + nl * PS + o0) = make_uint2(pack2<F16>(pv[0], pv[1]), pack2<F16>(pv[2], pv[3]));
            }
          }
          if (!IS_DV && own && grp == 0) {
            const float tot = rsum + __shfl_xor(rsum, 32);
            if (h == 0) rows[u * 32 + r] = tot;  // units above the diagonal publish zero
          }
        }
      }

      // ---- denominators (forward, own chunk = last source chunk, first group only); NTH/64 threads share a row
      if (!IS_DV && own && grp == 0) {
        __syncthreads();  // row sums visible
        constexpr int TPR = NTH / 64;  // threads per row: 8, 4, 2 or 1
        const int td = opaque(tid);
        const int t = td / TPR, part = td % TPR;
        const int seg = DHQK / TPR;
        const uint16_t* qrow = Ns + t * QS + part * seg;
        const float* np = nperm + part * seg;
        float dot = 0.f;
        for (int d = 0; d < seg; d += 8) {
          const uint4 qv = *(const uint4*)(qrow + d);
          const uint32_t qq[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
          for (int p = 0; p < 4; ++p) {
            dot += lo2<F16>(qq[p]) * np[d + 2 * p];
            dot += hi2<F16>(qq[p]) * np[d + 2 * p + 1];
          }
        }
#pragma unroll
        for (int o = TPR / 2; o > 0; o >>= 1) dot += __shfl_xor(dot, o);
        if (part == 0) {
          float nmax = 1.f, iv = 1.f;
          if (a.use_nrow) {
            float den = cs0[t] * dot;
#pragma unroll
            for (int ob4 = 0; ob4 < 4; ++ob4) den += rows[(2 * ob4 + (t >> 5)) * 32 + (t & 31)];
            const float mc = mcs[t];
            const float floor_v = a.sig_gate ? 1.f : __expf(-mc);
            nmax = fmaxf(fabsf(den), floor_v);
            iv = 1.f / (nmax + a.eps);
          }
          inv[t] = iv;
          a.nrow_out[gofs + n0 + t] = nmax;
          const int tg = t_base + n0 + t;
          if (tg < S) {
            if (a.n_out != nullptr) a.n_out[(size_t)bh * S + tg] = nmax;
            if (a.m_out != nullptr) a.m_out[(size_t)bh * S + tg] = mcs[t];
          }
        }
      }

      // ---- Out^T += Xw^T P over the live rows of the source chunk
      const int nv2 = nv + (nv & 1);
      for (int vs = 0; vs < nv2; vs += 2) {
        MLSTM_V_STEP(sA, ovA, orA, vs)
        MLSTM_V_STEP(sB, ovB, orB, vs + 1)
      }
    }

    // The next group's first state fragments travel during the epilogue (held across the score and value phases they
    // would cost the registers those need).  Unconditional: after the last group the fragments of that group are
    // requested once more, cache hits nobody waits for; a conditional load would be parked in scratch memory.
    MLSTM_LOAD_RING(min(grp + 1, NG - 1) * GW)
    // ---- optional head norm (forward only; the launcher admits it only when one group spans the whole value
    // dimension, so that this workgroup holds complete rows of H): with x = H_t, y = (x - mean) * rsqrt(var + eps) over
    // the DHHV columns ("layer"), or y = x * rsqrt(mean(x^2) + eps) ("rms").  Statistics in fp32 from the fp32
    // accumulators (sum and sum of squares; x = acc * iv, so both come from the raw accumulators); each lane owns one
    // position per 32-position block and a share of its columns, the shares of the waves meet in the slab buffer.  The
    // result is an affine map of the accumulator, y = acc * osc + osh, applied when the rows are rounded below.
    constexpr bool normed = !IS_DV && HEAD_NORM;
    float osc[2] = {1.f, 1.f}, osh[2] = {0.f, 0.f};
    if constexpr (normed) {
      const int le = opaque(lane);
      const int r = le & 31, h = le >> 5;
      float* red = (float*)Ts;  // [NWAVE][2][64]
      float p1[2], p2[2];
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int tl = 0; tl < NTG; ++tl)
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              const float x = acc[tl][mb][nb][i];
              s1 += x;
              s2 += x * x;
            }
        p1[nb] = s1 + __shfl_xor(s1, 32);
        p2[nb] = s2 + __shfl_xor(s2, 32);
      }
      __syncthreads();  // slab buffer free (last value slab consumed)
      if (h == 0) {
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
          red[wave * 128 + 32 * nb + r] = p1[nb];
          red[wave * 128 + 64 + 32 * nb + r] = p2[nb];
        }
      }
      __syncthreads();
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        float t1 = 0.f, t2 = 0.f;
#pragma unroll
        for (int w = 0; w < NWAVE; ++w) {
          t1 += red[w * 128 + 32 * nb + r];
          t2 += red[w * 128 + 64 + 32 * nb + r];
        }
        const float iv = inv[32 * nb + r];
        const float ex = t1 * iv * (1.f / (float)DHHV), ex2 = t2 * iv * iv * (1.f / (float)DHHV);
        const float mean = a.head_norm == 1 ? ex : 0.f;
        const float rstd = rsqrtf(fmaxf(ex2 - mean * mean, 0.f) + a.norm_eps);
        osc[nb] = iv * rstd;
        osh[nb] = -mean * rstd;
        const int tg = t_base + n0 + 32 * nb + r;
        if (wave == 0 && h == 0 && tg < S) {
          a.norm_mean[(size_t)bh * S + tg] = mean;
          a.norm_rstd[(size_t)bh * S + tg] = rstd;
        }
      }
    }
    // ---- epilogue: (normalise,) round, transpose through LDS, coalesced store.  The score block and the slab buffer
    // are both free now and lie next to each other: together they hold all 64 positions of a column tile, so a tile
    // costs two barriers.
    static_assert(64 * PS + t_region >= 64 * HS, "score block + slab buffer stage 64 output rows");
    uint16_t* const Os = Ps;
#pragma unroll
    for (int tl = 0; tl < NTG; ++tl) {
      uint16_t* Og = a.Out + (size_t)bh * S * DHHV + grp * GW + tl * WT;
      const int le = opaque(lane);
      const int r = le & 31, h = le >> 5;
      __syncthreads();  // staging area free (last value slab and score block consumed / previous tile stored; inv written)
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        const float iv = IS_DV ? 1.f : (normed ? osc[nb] : inv[32 * nb + r]);
        const float sh = normed ? osh[nb] : 0.f;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
          for (int g4 = 0; g4 < 4; ++g4) {
            const int w0 = m_wave + 32 * mb + 8 * g4 + 4 * h;
            *(uint2*)(Os + (32 * nb + r) * HS + w0) =
                make_uint2(pack2<F16>(acc[tl][mb][nb][4 * g4 + 0] * iv + sh, acc[tl][mb][nb][4 * g4 + 1] * iv + sh),
                           pack2<F16>(acc[tl][mb][nb][4 * g4 + 2] * iv + sh, acc[tl][mb][nb][4 * g4 + 3] * iv + sh));
          }
      }
      __syncthreads();
      constexpr int vec_per_row = WT / 8;
      for (int idx = opaque(tid); idx < 64 * vec_per_row; idx += NTH) {
        const int j = idx / vec_per_row, cv = idx % vec_per_row;
        const int t = t_base + n0 + j;
        // non-temporal: nobody in this launch reads the output, it should not evict shared operands from the L2
        if (t < S) __builtin_nontemporal_store(*(const u32x4*)(Os + j * HS + cv * 8), (u32x4*)(Og + (size_t)t * DHHV + cv * 8));
      }
    }
  }
#undef MLSTM_LOAD_RING
#undef MLSTM_STATE_FRAG
#undef MLSTM_LOAD_AT
#undef MLSTM_K_STEP
#undef MLSTM_V_STEP
}

template <int WT, int NTG, bool IS_DV, int PD, int MW, bool HEAD_NORM, bool F16>
__global__ __launch_bounds__(64 * (WT / MW))
    __attribute__((amdgpu_waves_per_eu(PAR_HV_WPE(WT, MW), PAR_HV_WPE(WT, MW)))) void par_hv_kernel(ParHvArgs a) {
  par_hv_body<WT, NTG, IS_DV, PD, MW, HEAD_NORM, F16>(a, xcd_block_id());  // the workgroups that share a kept state run on one XCD
}

template <int WT, int NTG, bool IS_DV, int PD, int MW, bool HEAD_NORM, bool F16>
static const char* launch_par_hv_hn(const ParHvArgs& a, int BH, hipStream_t stream) {
  constexpr int GW = WT * NTG;
  constexpr int VR = 8192 / GW;
  const int QS = a.DHQK + 8;
  const size_t n_region = (size_t)64 * QS;
  const size_t t_region = (128 * 72 > VR * (GW + 32)) ? 128 * 72 : VR * (GW + 32);
  const size_t smem = (n_region + 64 * 136 + t_region) * 2 + (size_t)(64 + 128 * 2 + 64 * 2 + 8 * 32 + a.DHQK + 64 * 2) * 4;
  if (smem > 160 * 1024) return "par_hv: DHQK too large for the LDS-resident tile";
  if ((size_t)a.S * (size_t)(a.DHHV > a.DHQK ? a.DHHV : a.DHQK) * 2 >= ((size_t)1 << 32))
    return "par_hv: one (batch, head) slab of an input exceeds 4 GiB";
  if (hipFuncSetAttribute((const void*)par_hv_kernel<WT, NTG, IS_DV, PD, MW, HEAD_NORM, F16>, hipFuncAttributeMaxDynamicSharedMemorySize,
                          (int)smem) != hipSuccess)
    return "par_hv: cannot raise the dynamic LDS limit";
  dim3 grid(2, a.NC, BH);
  hipLaunchKernelGGL((par_hv_kernel<WT, NTG, IS_DV, PD, MW, HEAD_NORM, F16>), grid, dim3(64 * (WT / MW)), smem, stream, a);
  return nullptr;
}

template <int WT, int NTG, bool IS_DV, int PD, int MW>
static const char* launch_par_hv_pd(const ParHvArgs& a, int BH, hipStream_t stream) {
  if constexpr (!IS_DV) {
    if (a.head_norm != 0)
      return a.f16 ? launch_par_hv_hn<WT, NTG, IS_DV, PD, MW, true, true>(a, BH, stream)
                   : launch_par_hv_hn<WT, NTG, IS_DV, PD, MW, true, false>(a, BH, stream);
  }
  return a.f16 ? launch_par_hv_hn<WT, NTG, IS_DV, PD, MW, false, true>(a, BH, stream)
               : launch_par_hv_hn<WT, NTG, IS_DV, PD, MW, false, false>(a, BH, stream);
}

template <int WT, int NTG, bool IS_DV>
static const char* launch_par_hv_t(const ParHvArgs& a, int BH, hipStream_t stream) {
  // eight steps ahead (64 registers of fragments in flight per lane) measured 8 % faster than four at 256/512
  constexpr int MW = WT == 256 ? 32 : 64;
  if (a.DHQK % 128 == 0) return launch_par_hv_pd<WT, NTG, IS_DV, 8, MW>(a, BH, stream);
  return launch_par_hv_pd<WT, NTG, IS_DV, 4, MW>(a, BH, stream);
}

template <bool IS_DV>
static const char* launch_par_hv_d(const ParHvArgs& a, int BH, hipStream_t stream) {
  if (a.DHHV % 512 == 0) return launch_par_hv_t<256, 2, IS_DV>(a, BH, stream);
  if (a.DHHV % 256 == 0) return launch_par_hv_t<256, 1, IS_DV>(a, BH, stream);
  if (a.DHHV % 128 == 0) return launch_par_hv_t<128, 1, IS_DV>(a, BH, stream);
  return launch_par_hv_t<64, 1, IS_DV>(a, BH, stream);
}

// one workgroup holds complete rows of H only when a single group of column tiles spans the value dimension
bool par_hv_head_norm_supported(int DHHV) { return DHHV == 64 || DHHV == 128 || DHHV == 256 || DHHV == 512; }

const char* launch_par_hv(const ParHvArgs& a, int BH, bool is_dv, hipStream_t stream) {
  if (a.DHQK % 64 != 0 || a.DHHV % 64 != 0) return "par_hv: DHQK and DHHV must be multiples of 64";
  if (a.stride < 1 || a.stride > kMaxStateStride) return "par_hv: state stride out of range";
  if (a.head_norm != 0) {
    if (is_dv) return "par_hv: the head norm belongs to the forward output";
    if (a.head_norm != 1 && a.head_norm != 2) return "par_hv: unknown head norm code";
    if (!par_hv_head_norm_supported(a.DHHV)) return "par_hv: the fused head norm needs DHHV = 64, 128, 256 or 512";
    if (a.norm_mean == nullptr || a.norm_rstd == nullptr) return "par_hv: the head norm needs its mean / rstd outputs";
  }
  return is_dv ? launch_par_hv_d<true>(a, BH, stream) : launch_par_hv_d<false>(a, BH, stream);
}

}  // namespace mlstm
