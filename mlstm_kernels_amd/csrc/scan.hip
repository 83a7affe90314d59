// Inter-chunk state scan of the chunkwise mLSTM, forward (C states) and backward (dC states).
//
//   forward :  C_c  = gbar_c * C_{c-1} + K_c^T (abar . V_c)          c = 0 .. NC-1      (and n likewise)
//   backward:  dC_{c-1} = gbar_c * dC_c + Q_c^T (rho . dH_c)          c = NC-1 .. 0,
//              rho_t = bbar_t / sqrt(DHQK) / (nrow_t + eps)
//
// (mlstm_kernels/torch/chunkwise/native/fw.py:88-121 and bw.py:67-98 in the reference.)  Both are the same
// kernel: a (DHQK x DHHV) fp32 state tile stays in MFMA accumulators for the whole sequence; per chunk the
// tile is first written out as bf16 operand fragments (the state *before* the update, which is what the
// chunk-parallel kernels consume), then decayed and updated with X_c^T (rowscale . Y_c), contraction over
// the 128 chunk positions.  Both operands have the contraction index as their slow memory dimension, so
// both are staged row-major in LDS and fetched with the transposing 64-bit LDS read.
//
// The row scale is applied to Y (the narrower operand of the tile) in fp32 before rounding to bf16.  For the
// forward the scaled rows are split into a bf16 head and a bf16 remainder (two MFMAs) so that the final
// state keeps ~16 mantissa bits: a single bf16 rounding of abar*V leaves a relative error of about 1.5e-3
// in C, above the 1e-3 the state is specified to.
//
// Workgroups are renumbered so that all tiles of one (batch, head) run on the same XCD (the hardware deals
// consecutive workgroup ids round-robin to the 8 XCDs): the K/V rows every tile of a head re-reads then hit
// that XCD's L2 instead of going to HBM once per tile.
#include "common.h"
#include "kernels.h"

namespace mlstm {

constexpr int kGBlock = 256;  // chunks per refill of the decay-factor table in LDS

// A chunk is staged in 128 / PS pieces of PS positions (the contraction over positions is a plain sum): the
// smaller the piece, the smaller the LDS tiles and the prefetch registers, but the more barriers per chunk.
// Measured on MI355X (B=4, S=16384, NH=8, 256/512), forward / backward scan in ms:
//   four waves per 128 x 128 tile, one workgroup per CU (one wave per SIMD)      0.63 / 0.54
//   four waves, register cap for two workgroups per CU (backward: 78 KB LDS)     -    / 0.46
//   four waves, half-chunk pieces so that the forward fits twice per CU          0.66 / 0.55
//   eight waves per tile (64 x 32 per wave), one workgroup per CU                0.46 / 0.41   <- used
//   eight waves, two workgroups per CU (128 registers per lane)                  -    / 0.45
//   n recurrence shared out among the column tiles by lane masks / run by every column tile    0.51 / -    (0.48 used)
//   rows moved from global memory straight into LDS (global_load_lds_dwordx4 into a ring of four 64-position stages,
//   three stages ahead, XOR-swizzled tiles, one barrier per stage, rows scaled in place)   0.44 / 0.45
//     (bit-equal results; with parts switched off: loads alone 0.22, state stores 0.05, matrix work 0.10, in-place
//      scaling 0.04, barriers 0.04 -- the parts add up instead of overlapping, and waiting less for the loads does
//      not change the time)
//   two LDS buffers and two register sets, one barrier per chunk: the rows of chunk c+1 are scaled and written into
//   one buffer while chunk c is multiplied out of the other, chunk c+3 is requested meanwhile (unpadded swizzled
//   tiles, 141 KB)                                                0.37 / 0.36 without the n recurrence, 0.44 with it
//     (bit-equal states.  Per chunk a CU spends about 1500 cycles on LDS traffic, 1000 per SIMD on matrix
//      instructions and 1000 per SIMD on the conversion arithmetic of the staging; with two waves per SIMD these
//      mostly add up, whatever the order they are issued in: 2.2 us per chunk even at B = 1, where nothing else
//      uses the memory system)
// What pays is a second instruction stream per SIMD inside the same workgroup: the phases of a chunk (staging,
// state emission, matrix work) are serial per wave, and two waves per SIMD overlap one's LDS and conversion
// latencies with the other's matrix instructions.
#define SCAN_WPE(HILO_, WCOLS_) ((WCOLS_) == 64 && (HILO_) ? 1 : 2)
// WCOLS = value columns per wave (64 or 32): with 32 a 128 x 128 tile takes eight waves, two per SIMD, each with
// half the staging work and half the accumulators.
template <bool V>
struct BoolTag {
  static constexpr bool value = V;
};

template <int RT, int WT, bool HILO, int PS, int WCOLS, bool F16>
__global__ __launch_bounds__(64 * (RT / 64) * (WT / WCOLS))
    __attribute__((amdgpu_waves_per_eu(SCAN_WPE(HILO, WCOLS), SCAN_WPE(HILO, WCOLS)))) void scan_kernel(ScanArgs a) {
  constexpr int WC = WT / WCOLS;
  constexpr int NBW = WCOLS / 32;  // 32-column accumulator blocks per wave
  constexpr int NT = 64 * (RT / 64) * WC;
  constexpr int XS = RT + 32;  // LDS row strides (elements): consecutive rows start 16 banks (64 bytes) apart
  constexpr int YS = WT + 32;
  constexpr int XV = PS * RT / 8 / NT;   // 16-byte vectors per thread per piece
  constexpr int YV = PS * WT / 8 / NT;
  constexpr int NP = kChunk / PS;        // pieces per chunk
  constexpr int XROWS = NT / (RT / 8);   // rows covered by one sweep of the workgroup over X
  static_assert(XV >= 1 && YV >= 1 && PS % 16 == 0, "piece too small for this tile");
  extern __shared__ __align__(16) unsigned char smem_raw[];
  uint16_t* Xs = (uint16_t*)smem_raw;
  uint16_t* Yh = Xs + PS * XS;
  uint16_t* Yl = Yh + PS * YS;
  float* npart = (float*)(Yl + (HILO ? PS * YS : 0));  // [XROWS][RT] partial sums of the n update
  float* gl = npart + XROWS * RT;                       // [kGBlock] decay factors of the next chunks, in scan order
  float* scl = gl + kGBlock;                            // [2][128] row scales of the chunk being staged / the next one

  // the wave index is made scalar so that branches on it are scalar branches (accumulators stay in place)
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wr = wave / WC, wc = wave % WC;
  const int r = lane & 31, h = lane >> 5;
  // ---- XCD-aware renumbering: linear id -> (xcd, slot) -> contiguous range of ids per XCD
  int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
  {
    const int total = gridDim.x * gridDim.y * gridDim.z;
    if (total % 8 == 0) {
      const int lin = bx + gridDim.x * (by + gridDim.y * bz);
      const int virt = (lin % 8) * (total / 8) + lin / 8;
      bx = virt % gridDim.x;
      by = (virt / gridDim.x) % gridDim.y;
      bz = virt / (gridDim.x * gridDim.y);
    }
  }
  const int bh = bz;
  const int d_tile = bx * RT, w_tile = by * WT;
  const int d_wave = d_tile + wr * 64, w_wave = w_tile + wc * WCOLS;
  const int DHQK = a.DHQK, DHHV = a.DHHV, S = a.S, NC = a.NC;
  const size_t Sp = (size_t)NC * kChunk;

  f32x16 acc[2][NBW];
#pragma unroll
  for (int db = 0; db < 2; ++db)
#pragma unroll
    for (int wb = 0; wb < NBW; ++wb) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float v0 = 0.f;
        if (a.init != nullptr) {
          const int d = d_wave + 32 * db + 8 * (i / 4) + 4 * h + (i % 4);
          const int w = w_wave + 32 * wb + r;
          v0 = a.init[((size_t)bh * DHQK + d) * DHHV + w];
        }
        acc[db][wb][i] = v0;
      }
    }
  const bool do_n = (a.nstates != nullptr) && by == 0;
  float nval = 0.f;
  if (do_n && tid < RT && a.n_init != nullptr) nval = a.n_init[(size_t)bh * DHQK + d_tile + tid];

  const uint16_t* Xg = a.X + (size_t)bh * S * DHQK + d_tile;
  const uint16_t* Yg = a.Y + (size_t)bh * S * DHHV + w_tile;

  uint4 xr[XV], yr[YV];
  // Row scales (forward: abar_j; backward: bbar_t / sqrt(DHQK) / (nrow_t + eps)) go through a table in LDS instead of
  // one 4-byte load per staged vector: every thread fetches the factor of ONE row two chunks ahead (a single load
  // instruction per wave and chunk), the table entry is written while the chunk before it is staged.  The vector
  // memory path of the CU (64 bytes per clock for loads, stores and their address processing) is what the scan
  // queues on, so its instruction count matters.
  const int srow = tid & (kChunk - 1);
  const float* const nrow_or_dummy = a.nrow != nullptr ? a.nrow : a.scale_a;
  float s_raw = 0.f, s_nrm = 1.f;
  auto load_scales = [&](int c) {
    const int cc = min(max(c, 0), NC - 1);
    const int t = cc * kChunk + srow;
    s_raw = a.scale_a[bh * Sp + t];
    s_nrm = nrow_or_dummy[bh * Sp + t];
  };
  // The prefetch only LOADS: any arithmetic on a loaded value here would make the wave wait for the whole batch of
  // loads before it starts the matrix work they are meant to overlap with.
  auto prefetch = [&](int c, int piece) {
#pragma unroll
    for (int v = 0; v < XV; ++v) {
      const int idx = tid + v * NT;
      const int j = idx / (RT / 8), cv = idx % (RT / 8);
      const int t = c * kChunk + piece * PS + j;
      xr[v] = t < S ? *(const uint4*)(Xg + (size_t)t * DHQK + cv * 8) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int v = 0; v < YV; ++v) {
      const int idx = tid + v * NT;
      const int j = idx / (WT / 8), cv = idx % (WT / 8);
      const int t = c * kChunk + piece * PS + j;
      yr[v] = t < S ? *(const uint4*)(Yg + (size_t)t * DHHV + cv * 8) : make_uint4(0, 0, 0, 0);
    }
  };

  const int c_first = a.backward ? NC - 1 : 0, c_step = a.backward ? -1 : 1;
  // The remainder of the value operand serves the last state only, and chunk c enters the last state with the weight
  // W_c = product of the decay factors of the chunks after it (<= 1, non-increasing towards the start).  Chunks whose
  // weight is below 2^-8 are accumulated without the remainder: their rounding (2^-9 relative) then reaches the last
  // state at 2^-17 of its scale.  c_lo = first chunk that carries the remainder; every wave computes it for itself.
  int c_lo = 0;
  if constexpr (HILO) {
    if (!a.backward) {
      float carry = 1.f;
      int cnt = 0;
      for (int base = 0; base < NC; base += kWave) {
        const int cc = NC - 1 - (base + lane);                       // walking from the last chunk towards the first
        const float gv = cc >= 0 ? a.gbar[(size_t)bh * NC + cc] : 0.f;
        float incl = gv;                                            // inclusive prefix product over the lanes
#pragma unroll
        for (int o = 1; o < kWave; o <<= 1) {
          const float up = __shfl_up(incl, o);
          if (lane >= o) incl *= up;
        }
        float excl = __shfl_up(incl, 1);
        if (lane == 0) excl = 1.f;
        const bool need = cc >= 0 && carry * excl >= 0.00390625f;    // W_cc >= 2^-8
        const int n_need = __popcll(__ballot(need));
        cnt += n_need;
        if (n_need < kWave) break;                                   // weights only fall from here on
        carry *= __shfl(incl, kWave - 1);
      }
      c_lo = __builtin_amdgcn_readfirstlane(NC - cnt);
    }
  }
  // row scales of the first chunk straight into the table, those of the second chunk into the prefetch register
  {
    const int t = c_first * kChunk + srow;
    float sc0 = t < S ? a.scale_a[bh * Sp + t] : 0.f;
    if (a.backward) {
      sc0 *= a.qk_scale;
      if (a.nrow != nullptr) sc0 /= (a.nrow[bh * Sp + t] + a.eps);
    }
    if (tid < kChunk) scl[srow] = sc0;
  }
  load_scales(NC > 1 ? c_first + c_step : c_first);
  prefetch(c_first, 0);
  for (int hit = 0; hit < NC * NP; ++hit) {
    const int it = hit / NP, piece = hit % NP;
    const int c = c_first + it * c_step;
    // The decay factors come from LDS, a block of chunks at a time: read straight from global memory inside the
    // loop, the factor would sit behind the prefetch of the next chunk (loads complete in order) and the matrix
    // work would wait for the whole prefetch in every iteration.
    if (piece == 0 && (it & (kGBlock - 1)) == 0) {
      __syncthreads();
      for (int k = tid; k < kGBlock && it + k < NC; k += NT) gl[k] = a.gbar[(size_t)bh * NC + c + k * c_step];
      // visible after the barrier that follows the staging below
    }
    // ---- registers -> LDS (Y rows scaled in fp32, then rounded / split); partial sums of sum_j abar_j k_j
    const float* scur = scl + (it & 1) * kChunk + piece * PS;  // written while the previous chunk was staged
    const bool with_lo = HILO && c >= c_lo;                    // uniform over the workgroup
    if (piece == 0 && tid < kChunk) {
      // the next chunk's row scales (fetched two chunks ahead) into the other half of the table
      const int t = (c + c_step) * kChunk + srow;
      float sn = (it + 1 < NC && t < S) ? s_raw : 0.f;
      if (a.backward) {
        sn *= a.qk_scale;
        if (a.nrow != nullptr) sn /= (s_nrm + a.eps);
      }
      scl[((it + 1) & 1) * kChunk + srow] = sn;
    }
    float np[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int v = 0; v < XV; ++v) {
      const int idx = tid + v * NT;
      const int j = idx / (RT / 8), cv = idx % (RT / 8);
      *(uint4*)(Xs + j * XS + cv * 8) = xr[v];
      if (do_n) {
        const uint32_t in[4] = {xr[v].x, xr[v].y, xr[v].z, xr[v].w};
        const float xsc = scur[j];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          np[2 * p] += xsc * lo2<F16>(in[p]);
          np[2 * p + 1] += xsc * hi2<F16>(in[p]);
        }
      }
    }
    if (do_n) {
      // thread (row group tid/(RT/8), column vector tid%(RT/8)) holds the sum over its XV rows
      float* dst = npart + (tid / (RT / 8)) * RT + (tid % (RT / 8)) * 8;
      *(float4*)dst = make_float4(np[0], np[1], np[2], np[3]);
      *(float4*)(dst + 4) = make_float4(np[4], np[5], np[6], np[7]);
    }
#pragma unroll
    for (int v = 0; v < YV; ++v) {
      const int idx = tid + v * NT;
      const int j = idx / (WT / 8), cv = idx % (WT / 8);
      const uint32_t in[4] = {yr[v].x, yr[v].y, yr[v].z, yr[v].w};
      uint32_t hi[4], lo[4];
      const float sc = scur[j];
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const float e0 = lo2<F16>(in[p]) * sc;
        const float e1 = hi2<F16>(in[p]) * sc;
        hi[p] = pack2<F16>(e0, e1);
        if (HILO) lo[p] = pack2<F16>(e0 - lo2<F16>(hi[p]), e1 - hi2<F16>(hi[p]));
      }
      *(uint4*)(Yh + j * YS + cv * 8) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
      if (HILO) {
        if (with_lo) *(uint4*)(Yl + j * YS + cv * 8) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
      }
    }
    __syncthreads();
    if (hit + 1 < NC * NP) prefetch(piece + 1 < NP ? c : c + c_step, piece + 1 < NP ? piece + 1 : 0);
    if (piece == 0) load_scales(c + 2 * c_step);

    // ---- emit the state before this chunk's update as bf16 operand fragments, at the kept boundaries only: forward
    // the state before every stride-th chunk, backward the gradient of the state after the last chunk of every group
    // of `stride` chunks (and after the last chunk of the sequence); slot c / stride either way
    const bool keep = a.backward ? (c == NC - 1 || (c + 1) % a.stride == 0) : (c % a.stride == 0);
    if (piece == 0 && keep) {
      const size_t ND = DHQK / 16, NW = DHHV / 32;
      const size_t NCS = (size_t)(NC + a.stride - 1) / a.stride;
      uint4* st = (uint4*)a.states + ((size_t)bh * NCS + c / a.stride) * NW * ND * 64;
#pragma unroll
      for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int wb = 0; wb < NBW; ++wb) {
          const size_t W32 = (w_wave + 32 * wb) / 32, D16 = (d_wave + 32 * db) / 16;
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            uint4 f;
            f.x = pack2<F16>(acc[db][wb][8 * half + 0], acc[db][wb][8 * half + 1]);
            f.y = pack2<F16>(acc[db][wb][8 * half + 2], acc[db][wb][8 * half + 3]);
            f.z = pack2<F16>(acc[db][wb][8 * half + 4], acc[db][wb][8 * half + 5]);
            f.w = pack2<F16>(acc[db][wb][8 * half + 6], acc[db][wb][8 * half + 7]);
            // non-temporal: the fragments are read by a later kernel; kept out of the L2 they do not evict the K/V
            // rows the tiles of a head share
            const u32x4 fv = {f.x, f.y, f.z, f.w};
            __builtin_nontemporal_store(fv, (u32x4*)(st + (W32 * ND + D16 + half) * 64 + lane));
          }
        }
    }
    // ---- decay (once per chunk), then accumulate X^T (scale . Y) over the positions of this piece
    const float g = piece == 0 ? gl[it & (kGBlock - 1)] : 1.f;
    if (piece == 0) {
#pragma unroll
      for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int wb = 0; wb < NBW; ++wb) acc[db][wb] *= g;
    }

    const int q16 = (lane >> 4) & 1, i16 = lane & 15;
    const int krow = 8 * h + (i16 >> 2), ncol = 16 * q16 + 4 * (i16 & 3);
    // two copies of the loop (with and without the remainder) rather than a branch inside it: the accumulators stay
    // where they are either way
    auto multiply = [&](auto lo_tag) {
      constexpr bool LO = decltype(lo_tag)::value;
#pragma unroll
      for (int js = 0; js < PS / 16; ++js) {
        Frag A[2], Bh[NBW], Bl[NBW];
#pragma unroll
        for (int db = 0; db < 2; ++db) {
          const uint16_t* p = Xs + (16 * js + krow) * XS + (wr * 64 + 32 * db + ncol);
          A[db].d[0] = lds_read_tr16(p);
          A[db].d[1] = lds_read_tr16(p + 4 * XS);
        }
#pragma unroll
        for (int wb = 0; wb < NBW; ++wb) {
          const int o = (16 * js + krow) * YS + (wc * WCOLS + 32 * wb + ncol);
          Bh[wb].d[0] = lds_read_tr16(Yh + o);
          Bh[wb].d[1] = lds_read_tr16(Yh + o + 4 * YS);
          if (LO) {
            Bl[wb].d[0] = lds_read_tr16(Yl + o);
            Bl[wb].d[1] = lds_read_tr16(Yl + o + 4 * YS);
          }
        }
#pragma unroll
        for (int db = 0; db < 2; ++db)
#pragma unroll
          for (int wb = 0; wb < NBW; ++wb) {
            mfma32<F16>(acc[db][wb], A[db], Bh[wb]);
            if (LO) mfma32<F16>(acc[db][wb], A[db], Bl[wb]);
          }
      }
    };
    if (with_lo) multiply(BoolTag<HILO>{});
    else multiply(BoolTag<false>{});
    // ---- normaliser vector (forward, first column tile only): n = gbar n + sum_j abar_j k_j
    if (do_n && tid < RT) {
      if (piece == 0) a.nstates[((size_t)bh * NC + c) * DHQK + d_tile + tid] = nval;
      float s = 0.f;
#pragma unroll
      for (int g2 = 0; g2 < XROWS; ++g2) s += npart[g2 * RT + tid];
      nval = g * nval + s;
    }
    __syncthreads();
  }
  if (a.final_out != nullptr) {
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int wb = 0; wb < NBW; ++wb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int d = d_wave + 32 * db + 8 * (i / 4) + 4 * h + (i % 4);
          const int w = w_wave + 32 * wb + r;
          a.final_out[((size_t)bh * DHQK + d) * DHHV + w] = acc[db][wb][i];
        }
  }
  if (do_n && tid < RT && a.n_final != nullptr) a.n_final[(size_t)bh * DHQK + d_tile + tid] = nval;
}

template <int RT, int WT, bool HILO, bool F16>
static const char* launch_scan_f(const ScanArgs& a, int BH, hipStream_t stream) {
  constexpr int WCOLS = 32;
  constexpr int NT = 64 * (RT / 64) * (WT / WCOLS);
  constexpr int XROWS = NT / (RT / 8);
  constexpr int PS = 128;
  const size_t smem = (size_t)PS * (RT + 32) * 2 + (size_t)PS * (WT + 32) * 2 * (HILO ? 2 : 1) +
                      (size_t)(XROWS * RT + kGBlock + 2 * kChunk) * 4;
  if (hipFuncSetAttribute((const void*)scan_kernel<RT, WT, HILO, PS, WCOLS, F16>, hipFuncAttributeMaxDynamicSharedMemorySize,
                          (int)smem) != hipSuccess)
    return "scan: cannot raise the dynamic LDS limit";
  dim3 grid(a.DHQK / RT, a.DHHV / WT, BH);
  hipLaunchKernelGGL((scan_kernel<RT, WT, HILO, PS, WCOLS, F16>), grid, dim3(NT), smem, stream, a);
  return nullptr;
}

template <int RT, int WT, bool HILO>
static const char* launch_scan_t(const ScanArgs& a, int BH, hipStream_t stream) {
  return a.f16 ? launch_scan_f<RT, WT, HILO, true>(a, BH, stream) : launch_scan_f<RT, WT, HILO, false>(a, BH, stream);
}

const char* launch_scan(const ScanArgs& a, int BH, bool hilo, hipStream_t stream) {
  if (a.DHQK % 64 != 0 || a.DHHV % 64 != 0) return "scan: DHQK and DHHV must be multiples of 64";
  if (a.stride < 1 || a.stride > kMaxStateStride) return "scan: state stride out of range";
  const bool r128 = a.DHQK % 128 == 0, w128 = a.DHHV % 128 == 0;
  if (hilo) {
    if (r128 && w128) return launch_scan_t<128, 128, true>(a, BH, stream);
    if (r128) return launch_scan_t<128, 64, true>(a, BH, stream);
    if (w128) return launch_scan_t<64, 128, true>(a, BH, stream);
    return launch_scan_t<64, 64, true>(a, BH, stream);
  }
  if (r128 && w128) return launch_scan_t<128, 128, false>(a, BH, stream);
  if (r128) return launch_scan_t<128, 64, false>(a, BH, stream);
  if (w128) return launch_scan_t<64, 128, false>(a, BH, stream);
  return launch_scan_t<64, 64, false>(a, BH, stream);
}

}  // namespace mlstm
