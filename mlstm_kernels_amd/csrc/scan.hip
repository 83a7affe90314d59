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
// Two kernels: scan_roles_kernel (below, second) without the remainder -- the training forward, every backward scan,
// and of a forward that returns the fp32 last state the chunks whose rounding no longer shows in it -- and scan_kernel
// with the head + remainder split for the rest of such a forward (two launches; the state passes from one to the
// other in the caller's last-state buffers).  Same tiling, same arithmetic, same results.
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
// scan_kernel: eight waves per 128 x 128 tile (64 x 32 per wave), one workgroup per CU.  scan_roles_kernel: two LDS
// buffers and sixteen waves in two roles -- eight producer waves fetch, scale and stage the rows of chunk c+1 while
// eight consumer waves do the fragment reads and matrix instructions of chunk c (one barrier per chunk); the
// normaliser recurrence rides as three more operand columns on the consumers' matrix pipe.
// What pays is more instruction streams per SIMD inside the same workgroup: the phases of a chunk (staging, state
// emission, matrix work) are serial per wave; two waves per SIMD overlap one's LDS and conversion latencies with the
// other's matrix instructions, and four waves in two roles keep the conversion arithmetic and the matrix
// instructions in different waves altogether.
// The remainder of the value operand serves the last state only, and chunk c enters the last state with the weight
// W_c = product of the decay factors of the chunks after it (<= 1, non-increasing towards the start).  Chunks whose
// weight is below 2^-8 are accumulated without the remainder: their rounding (2^-9 relative) then reaches the last
// state at 2^-17 of its scale.  Returns the first chunk that carries the remainder (at most NC - 1); every wave
// computes it for itself, and every kernel that needs it gets the same value.
__device__ __forceinline__ int first_remainder_chunk(const float* gbar_bh, int NC, int lane) {
  float carry = 1.f;
  int cnt = 0;
  for (int base = 0; base < NC; base += kWave) {
    const int cc = NC - 1 - (base + lane);                       // walking from the last chunk towards the first
    const float gv = cc >= 0 ? gbar_bh[cc] : 0.f;
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
  return __builtin_amdgcn_readfirstlane(NC - cnt);
}

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
        const float* init = a.part == 2 ? a.final_out : a.init;  // part 2 continues from the first launch's state
        if (init != nullptr) {
          const int d = d_wave + 32 * db + 8 * (i / 4) + 4 * h + (i % 4);
          const int w = w_wave + 32 * wb + r;
          v0 = init[((size_t)bh * DHQK + d) * DHHV + w];
        }
        acc[db][wb][i] = v0;
      }
    }
  const bool do_n = (a.nstates != nullptr) && by == 0;
  float nval = 0.f;
  {
    const float* n_init = a.part == 2 ? a.n_final : a.n_init;
    if (do_n && tid < RT && n_init != nullptr) nval = n_init[(size_t)bh * DHQK + d_tile + tid];
  }

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

  const int c_first_all = a.backward ? NC - 1 : 0, c_step = a.backward ? -1 : 1;
  // c_lo = first chunk that carries the remainder of the value operand
  int c_lo = 0;
  if constexpr (HILO) {
    if (!a.backward) c_lo = a.all_remainder ? 0 : first_remainder_chunk(a.gbar + (size_t)bh * NC, NC, lane);
  }
  // part 2 of a forward scan in two launches: the chunks from c_lo on, continuing from the state the first launch left
  // in final_out / n_final (loaded above)
  const int c_first = a.part == 2 ? c_lo : c_first_all;
  const int NCR = a.part == 2 ? NC - c_lo : NC;  // chunks this launch runs
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
  load_scales(NCR > 1 ? c_first + c_step : c_first);
  prefetch(c_first, 0);
  for (int hit = 0; hit < NCR * NP; ++hit) {
    const int it = hit / NP, piece = hit % NP;
    const int c = c_first + it * c_step;
    // The decay factors come from LDS, a block of chunks at a time: read straight from global memory inside the
    // loop, the factor would sit behind the prefetch of the next chunk (loads complete in order) and the matrix
    // work would wait for the whole prefetch in every iteration.
    if (piece == 0 && (it & (kGBlock - 1)) == 0) {
      __syncthreads();
      for (int k = tid; k < kGBlock && it + k < NCR; k += NT) gl[k] = a.gbar[(size_t)bh * NC + c + k * c_step];
      // visible after the barrier that follows the staging below
    }
    // ---- registers -> LDS (Y rows scaled in fp32, then rounded / split); partial sums of sum_j abar_j k_j
    const float* scur = scl + (it & 1) * kChunk + piece * PS;  // written while the previous chunk was staged
    const bool with_lo = HILO && c >= c_lo;                    // uniform over the workgroup
    if (piece == 0 && tid < kChunk) {
      // the next chunk's row scales (fetched two chunks ahead) into the other half of the table
      const int t = (c + c_step) * kChunk + srow;
      float sn = (it + 1 < NCR && t < S) ? s_raw : 0.f;
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
    if (hit + 1 < NCR * NP) prefetch(piece + 1 < NP ? c : c + c_step, piece + 1 < NP ? piece + 1 : 0);
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
      if (piece == 0) {
        // three partial vectors per chunk (the consumer adds them up): this kernel keeps the whole sum in the first
        float* dst = a.nstates + ((size_t)bh * NC + c) * 3 * DHQK + d_tile + tid;
        dst[0] = nval;
        dst[DHQK] = 0.f;
        dst[2 * DHQK] = 0.f;
      }
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

// ---------------------------------------------------------------------------------------------------------------
// scan_roles_kernel: software pipeline over whole chunks with two LDS buffers and, per producer wave, two register
// sets.  While chunk c is multiplied out of one buffer, the rows of chunk c+1 (fetched two chunks earlier) are scaled,
// rounded and written into the other buffer, and the rows of chunk c+3 are requested into the register set this
// frees: ONE barrier per chunk, a global load has two chunk periods to arrive.  The tiles are unpadded (two buffers
// of a 128 x 128 tile pair fill 128 KB) and XOR-swizzled in 16-byte units so that the four rows a transposing read
// touches per half wave fall into four different 64-byte bank groups.
namespace {
template <int U>  // 16-byte units per tile row
__device__ __forceinline__ int scan_swz(int row) {
  return U == 8 ? ((row >> 1) & 1) << 2 : (row & 3) << 2;
}
struct ScanTrOff {
  int lo, hi;
};
// per-lane element offsets of the two transposing reads of a fragment (rows k0 + 8h .. +3 and +4 .. +7 of the
// contraction index, columns col0 .. col0+31) in a tile with ROWLEN elements per row; k0 is a multiple of 16, so the
// swizzle of the rows does not depend on it
template <int ROWLEN>
__device__ __forceinline__ ScanTrOff scan_tr_offsets(int col0, int lane) {
  const int q16 = (lane >> 4) & 1, i16 = lane & 15, h = lane >> 5;
  const int krow = 8 * h + (i16 >> 2);
  const int col = col0 + 16 * q16 + 4 * (i16 & 3);
  const int unit = col >> 3, sub = col & 7;
  ScanTrOff o;
  o.lo = krow * ROWLEN + ((unit ^ scan_swz<ROWLEN / 8>(krow)) << 3) + sub;
  o.hi = (krow + 4) * ROWLEN + ((unit ^ scan_swz<ROWLEN / 8>(krow + 4)) << 3) + sub;
  return o;
}
template <int ROWLEN>
__device__ __forceinline__ Frag scan_tr_frag(const uint16_t* tile, int k0, const ScanTrOff& o) {
  Frag f;
  f.d[0] = lds_read_tr16(tile + k0 * ROWLEN + o.lo);
  f.d[1] = lds_read_tr16(tile + k0 * ROWLEN + o.hi);
  return f;
}
}  // namespace

// The consumer role of the scan kernel (see there).  NDB = 0 or 1: this wave also carries the normaliser vector of the
// first or second 32 of its 64 state rows, NDB = -1: it does not (copies of the role rather than a branch around matrix
// instructions, which would make the compiler keep those accumulators in scratch memory).
template <int RT, int WT, bool F16, int NDB>
__device__ __forceinline__ void scan_consumer(const ScanArgs& a, const uint16_t* bufs, const float* gl, const uint16_t* nB,
                                              int wave, int lane, int bh, int d_tile, int w_tile, int n_run) {
  constexpr int c_lo = 0;  // (no remainder operand in this kernel)
  constexpr bool HILO = false;
  constexpr int WC = WT / 32;
  constexpr int PS = HILO ? 64 : 128;
  constexpr int NP = kChunk / PS;
  constexpr int XELEMS = PS * RT, YELEMS = PS * WT;
  constexpr int BUF = XELEMS + YELEMS * (HILO ? 2 : 1);
  const int DHQK = a.DHQK, DHHV = a.DHHV, NC = a.NC;
  const int total = n_run * NP;  // n_run: chunks this launch runs
  const int c_first = a.backward ? NC - 1 : 0, c_step = a.backward ? -1 : 1;
  constexpr bool WITH_N = NDB >= 0;
  constexpr int DB = WITH_N ? NDB : 0;
  auto refill_due = [&](int p) { return p % NP == 0 && p / NP > 0 && ((p / NP) & (kGBlock - 1)) == 0; };
  const int wr = wave / WC, wc = wave % WC;
  const int r = lane & 31, h = lane >> 5;
  const int d_wave = d_tile + wr * 64, w_wave = w_tile + wc * 32;
  f32x16 acc[2];
#pragma unroll
  for (int db = 0; db < 2; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float v0 = 0.f;
      if (a.init != nullptr) {
        const int d = d_wave + 32 * db + 8 * (i / 4) + 4 * h + (i % 4);
        v0 = a.init[((size_t)bh * DHQK + d) * DHHV + w_wave + r];
      }
      acc[db][i] = v0;
    }
  // normaliser vector: the waves of the first 32 value columns of the first column tile carry it as three partial
  // columns (lanes r = 0, 1, 2) of one more accumulator pair, see write_n_operand
  f32x16 accn;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    float v0 = 0.f;
    if (WITH_N && a.n_init != nullptr && r == 0) v0 = a.n_init[(size_t)bh * DHQK + d_wave + 32 * DB + 8 * (i / 4) + 4 * h + (i % 4)];
    accn[i] = v0;
  }
  const ScanTrOff offA0 = scan_tr_offsets<RT>(wr * 64, lane);
  const ScanTrOff offA1 = scan_tr_offsets<RT>(wr * 64 + 32, lane);
  const ScanTrOff offB = scan_tr_offsets<WT>(wc * 32, lane);
  __syncthreads();  // the producers' prologue barrier
  for (int p = 0; p < total; ++p) {
    const int it = p / NP, piece = p % NP;
    const int c = c_first + it * c_step;
    if (refill_due(p)) __syncthreads();
    __syncthreads();  // piece p staged by the producers
    if (piece == 0) {
      // ---- the state before this chunk's update as operand fragments, at the kept boundaries only: forward the
      // state before every stride-th chunk, backward the gradient of the state after the last chunk of every group
      // of `stride` chunks (and after the last chunk of the sequence); slot c / stride either way
      const bool keep = a.backward ? (c == NC - 1 || (c + 1) % a.stride == 0) : (c % a.stride == 0);
      if (keep) {
        const size_t ND = DHQK / 16, NWB = DHHV / 32;
        const size_t NCS = (size_t)(NC + a.stride - 1) / a.stride;
        u32x4* st = (u32x4*)a.states + ((size_t)bh * NCS + c / a.stride) * NWB * ND * 64;
#pragma unroll
        for (int db = 0; db < 2; ++db) {
          const size_t W32 = w_wave / 32, D16 = (d_wave + 32 * db) / 16;
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            u32x4 f;
#pragma unroll
            for (int e = 0; e < 4; ++e) f[e] = pack2<F16>(acc[db][8 * half + 2 * e], acc[db][8 * half + 2 * e + 1]);
            // non-temporal: the fragments are read by a later kernel; kept out of the L2 they do not evict the K/V
            // rows the tiles of a head share
            __builtin_nontemporal_store(f, st + (W32 * ND + D16 + half) * 64 + lane);
          }
        }
      }
      const float g = gl[it & (kGBlock - 1)];
      acc[0] *= g;
      acc[1] *= g;
      if (WITH_N) {
        // n before this chunk, as its three partial vectors [3][DHQK] (the consumer of the states adds them up)
        if (r < 3) {
          float* dst = a.nstates + (((size_t)bh * NC + c) * 3 + r) * DHQK + d_wave + 32 * DB + 4 * h;
#pragma unroll
          for (int g4 = 0; g4 < 4; ++g4)
            *(float4*)(dst + 8 * g4) = make_float4(accn[4 * g4], accn[4 * g4 + 1], accn[4 * g4 + 2], accn[4 * g4 + 3]);
        }
        accn *= g;
      }
    }
    // ---- accumulate X^T (scale . Y) over the positions of this piece; two copies of the loop (with and without
    // the remainder) rather than a branch inside it: the accumulators stay where they are either way
    const uint16_t* Xs = bufs + (p & 1) * BUF;
    const uint16_t* Yh = Xs + XELEMS;
    const uint16_t* Yl = Yh + YELEMS;
    const uint16_t* nBp = nB + (it % 3) * (kChunk * 3) + (piece * (PS / 8) + h) * 24 + min(r, 2) * 8;
    auto multiply_step = [&](auto lo_tag, int js) {
      constexpr bool LO = decltype(lo_tag)::value;
      const Frag A0 = scan_tr_frag<RT>(Xs, 16 * js, offA0), A1 = scan_tr_frag<RT>(Xs, 16 * js, offA1);
      const Frag Bh = scan_tr_frag<WT>(Yh, 16 * js, offB);
      mfma32<F16>(acc[0], A0, Bh);
      mfma32<F16>(acc[1], A1, Bh);
      if (WITH_N) {
        Frag Bn;
        Bn.u = *(const uint4*)(nBp + js * 48);
        if (r >= 3) Bn.u = make_uint4(0, 0, 0, 0);
        mfma32<F16>(accn, DB == 0 ? A0 : A1, Bn);
      }
      if (LO) {
        const Frag Bl = scan_tr_frag<WT>(Yl, 16 * js, offB);
        mfma32<F16>(acc[0], A0, Bl);
        mfma32<F16>(acc[1], A1, Bl);
      }
    };
    auto multiply = [&](auto lo_tag) {
      if constexpr (decltype(lo_tag)::value) {
        // with the remainder operand a step holds four fragments: two steps in flight fit the 128 registers of a wave
#pragma unroll 2
        for (int js = 0; js < PS / 16; ++js) multiply_step(lo_tag, js);
      } else {
#pragma unroll
        for (int js = 0; js < PS / 16; ++js) multiply_step(lo_tag, js);
      }
    };
    if (HILO && c >= c_lo) multiply(BoolTag<HILO>{});
    else multiply(BoolTag<false>{});
  }
  if (a.final_out != nullptr) {
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int d = d_wave + 32 * db + 8 * (i / 4) + 4 * h + (i % 4);
        a.final_out[((size_t)bh * DHQK + d) * DHHV + w_wave + r] = acc[db][i];
      }
  }
  if (WITH_N && a.n_final != nullptr) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      // the three partial columns live in lanes r = 0, 1, 2 of either half wave
      const float x = accn[i];
      const float sum = __shfl(x, 32 * h) + __shfl(x, 32 * h + 1) + __shfl(x, 32 * h + 2);
      if (r == 0) a.n_final[(size_t)bh * DHQK + d_wave + 32 * DB + 8 * (i / 4) + 4 * h + (i % 4)] = sum;
    }
  }
}

// RT x WT state tile.  HILO: the scaled value rows are split into a 16-bit head and a 16-bit remainder (pieces of 64
// positions), otherwise rounded once (pieces of 128 positions).
//
// The workgroup has two kinds of waves, NWC of each: CONSUMER waves own a 64 x 32 block of the state tile in their
// accumulators and do nothing but fragment reads, matrix instructions, the decay and the emission of the state;
// PRODUCER waves fetch the rows, scale / round / split them and write them into the LDS buffer the consumers will read
// next, keep the normaliser vector and the scale table.  The two instruction streams of a SIMD that limit each other
// when every wave does everything (conversion arithmetic against matrix instructions) then belong to different waves
// and overlap; four waves per SIMD instead of two.
template <int RT, int WT, bool F16>
__global__ __launch_bounds__(128 * (RT / 64) * (WT / 32)) void scan_roles_kernel(ScanArgs a) {
  constexpr bool HILO = false;  // the remainder split of the value operand is the other kernel's
  constexpr int WC = WT / 32;
  constexpr int NWC = (RT / 64) * WC;     // consumer waves (and as many producer waves)
  constexpr int NTP = 64 * NWC;           // producer threads
  constexpr int PS = HILO ? 64 : 128;     // positions per piece
  constexpr int NP = kChunk / PS;         // pieces per chunk
  constexpr int XU = RT / 8, YU = WT / 8; // 16-byte units per row
  constexpr int XV = PS * XU / NTP;       // 16-byte vectors per producer thread per piece
  constexpr int YV = PS * YU / NTP;
  constexpr int XRG = NTP / XU;           // rows one sweep of the producers covers (X); a thread's rows are XRG apart
  constexpr int YRG = NTP / YU;
  constexpr int XELEMS = PS * RT, YELEMS = PS * WT;
  constexpr int BUF = XELEMS + YELEMS * (HILO ? 2 : 1);  // elements per LDS buffer
  static_assert(XV >= 1 && YV >= 1 && XRG % 4 == 0 && YRG % 4 == 0, "tile shape does not fit the staging pattern");
  extern __shared__ __align__(16) unsigned char smem_raw[];
  uint16_t* bufs = (uint16_t*)smem_raw;                 // [2][X | Yh | Yl]
  float* gl = (float*)(bufs + 2 * BUF);                 // [kGBlock] decay factors of the next chunks, in scan order
  float* scl = gl + kGBlock;                            // [2][128] row scales, by chunk parity
  uint16_t* nB = (uint16_t*)(scl + 2 * kChunk);         // [3][128 / 8][3][8] the row scales as a matrix operand (below)

  // the wave index is made scalar so that branches on it are scalar branches
  const int lane = threadIdx.x & 63, wave_all = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const bool producer = wave_all < NWC;
  const int wave = producer ? wave_all : wave_all - NWC;
  const int tid = wave * 64 + lane;                     // index inside the own group of waves
  const BlockId blk = xcd_block_id();  // all tiles of one (batch, head) on one XCD: they share its K/V rows in the L2
  const int bh = blk.z;
  const int d_tile = blk.x * RT, w_tile = blk.y * WT;
  const int DHQK = a.DHQK, DHHV = a.DHHV, S = a.S, NC = a.NC;
  const size_t Sp = (size_t)NC * kChunk;
  // part 1 of a forward scan in two launches: only the chunks before the first one that carries the remainder of the
  // value operand; the state reached there is handed over in final_out / n_final
  const int n_run = a.part == 1 ? (a.all_remainder ? 0 : first_remainder_chunk(a.gbar + (size_t)bh * NC, NC, lane)) : NC;
  const int total = n_run * NP;
  const int c_first = a.backward ? NC - 1 : 0, c_step = a.backward ? -1 : 1;

  constexpr int c_lo = 0;  // (no remainder operand in this kernel)
  // Both kinds of waves pass the same barriers: one after the prologue, one per piece, and one more before every
  // refill of the decay table (every kGBlock chunks).
  auto refill_due = [&](int p) { return p % NP == 0 && p / NP > 0 && ((p / NP) & (kGBlock - 1)) == 0; };

  if (producer) {
    // ======================================================================================= producer waves
    const bool do_n = (a.nstates != nullptr) && blk.y == 0;
    const uint16_t* Xg = a.X + (size_t)bh * S * DHQK + d_tile + (tid % XU) * 8;
    const uint16_t* Yg = a.Y + (size_t)bh * S * DHHV + w_tile + (tid % YU) * 8;
    const int xrow = tid / XU, yrow = tid / YU;  // first row of this thread inside a piece; further rows XRG / YRG apart
    // LDS store offsets of the first row (elements); the rows of a thread are a multiple of 4 apart: same swizzle
    const int xst = xrow * RT + (((tid % XU) ^ scan_swz<XU>(xrow)) << 3);
    const int yst = yrow * WT + (((tid % YU) ^ scan_swz<YU>(yrow)) << 3);
    auto piece_t0 = [&](int p) { return (c_first + (p / NP) * c_step) * kChunk + (p % NP) * PS; };

    // ---- row scales (forward: abar_j; backward: bbar_t / sqrt(DHQK) / (nrow_t + eps)) go through a table in LDS:
    // every thread fetches the factor of ONE row of a chunk three chunks before that chunk is staged (first in its
    // batch of loads, so that waiting for it does not wait for the rows requested with it) and writes the table entry
    // one chunk later; positions past the end of the sequence get 0 and so neither feed the state nor the normaliser.
    const int srow = tid & (kChunk - 1);
    const float* const nrow_or_dummy = a.nrow != nullptr ? a.nrow : a.scale_a;
    float s_raw = 0.f, s_nrm = 1.f;
    auto load_scales = [&](int c) {  // c: chunk index in memory order, clamped
      const int cc = min(max(c, 0), NC - 1);
      s_raw = a.scale_a[bh * Sp + cc * kChunk + srow];
      s_nrm = nrow_or_dummy[bh * Sp + cc * kChunk + srow];
    };
    auto scale_value = [&](int c) {  // the table entry of row srow of chunk c from the fetched values
      float sn = (c >= 0 && c < NC && c * kChunk + srow < S) ? s_raw : 0.f;
      if (a.backward) {
        sn *= a.qk_scale;
        if (a.nrow != nullptr) sn /= (s_nrm + a.eps);
      }
      return sn;
    };

    // The normaliser recurrence n_c = gbar_c n_{c-1} + sum_j abar_j k_j rides on the matrix pipe of the consumers: the
    // row scale of every position, split exactly into three 16-bit parts, forms three columns of a B operand
    // (position 8b + e of a chunk, part r, at [b][r][e]); K^T times it gives sum_j abar_j k_j in three partial columns
    // whose sum carries 24 bits of every abar_j.  Slot c % 3: written two chunks before chunk c is multiplied.
    auto write_n_operand = [&](int it_of_chunk, float sn) {
      uint16_t* dst = nB + (it_of_chunk % 3) * (kChunk * 3) + (srow >> 3) * 24 + (srow & 7);
      const uint16_t p0 = f32_to_elem<F16>(sn);
      const float r1 = sn - elem_to_f32<F16>(p0);
      const uint16_t p1 = f32_to_elem<F16>(r1);
      const uint16_t p2 = f32_to_elem<F16>(r1 - elem_to_f32<F16>(p1));
      dst[0] = p0;
      dst[8] = p1;
      dst[16] = p2;
    };

    // two register sets, by piece parity (macros, not lambdas: with the arrays captured by reference the compiler keeps
    // them in scratch memory)
    u32x4 xr0[XV], yr0[YV], xr1[XV], yr1[YV];
    // The prefetch only LOADS: any arithmetic on a loaded value here would make the wave wait for the whole batch.
#define MLSTM_SCAN_PREFETCH(SET, p_)                                                                             \
  {                                                                                                              \
    const int t0_ = piece_t0(p_);                                                                                \
    _Pragma("unroll") for (int v = 0; v < XV; ++v) {                                                             \
      /* rows past the end re-read the last row; their scale is 0 */                                             \
      const int t = min(t0_ + xrow + v * XRG, S - 1);                                                            \
      xr##SET[v] = *(const u32x4*)(Xg + (size_t)t * DHQK);                                                       \
    }                                                                                                            \
    _Pragma("unroll") for (int v = 0; v < YV; ++v) {                                                             \
      const int t = min(t0_ + yrow + v * YRG, S - 1);                                                            \
      yr##SET[v] = *(const u32x4*)(Yg + (size_t)t * DHHV);                                                       \
    }                                                                                                            \
  }
    // registers -> LDS buffer `bi_` (Y rows scaled in fp32, then rounded / split)
#define MLSTM_SCAN_STAGE(SET, p_, bi_)                                                                           \
  {                                                                                                              \
    const int c_ = c_first + ((p_) / NP) * c_step, piece_ = (p_) % NP;                                           \
    uint16_t* Xs = bufs + (bi_) * BUF;                                                                           \
    uint16_t* Yh = Xs + XELEMS;                                                                                  \
    uint16_t* Yl = Yh + YELEMS;                                                                                  \
    const float* scur = scl + (((p_) / NP) & 1) * kChunk + piece_ * PS;                                          \
    const bool with_lo = HILO && c_ >= c_lo; /* uniform over the workgroup */                                    \
    _Pragma("unroll") for (int v = 0; v < XV; ++v) *(u32x4*)(Xs + xst + v * XRG * RT) = xr##SET[v];              \
    _Pragma("unroll") for (int v = 0; v < YV; ++v) {                                                             \
      const uint32_t in[4] = {yr##SET[v][0], yr##SET[v][1], yr##SET[v][2], yr##SET[v][3]};                       \
      uint32_t hi[4], lo[4];                                                                                     \
      const float sc = scur[yrow + v * YRG];                                                                     \
      _Pragma("unroll") for (int e = 0; e < 4; ++e) {                                                            \
        const float e0 = lo2<F16>(in[e]) * sc;                                                                   \
        const float e1 = hi2<F16>(in[e]) * sc;                                                                   \
        hi[e] = pack2<F16>(e0, e1);                                                                              \
        if (HILO) lo[e] = pack2<F16>(e0 - lo2<F16>(hi[e]), e1 - hi2<F16>(hi[e]));                                \
      }                                                                                                          \
      *(uint4*)(Yh + yst + v * YRG * WT) = make_uint4(hi[0], hi[1], hi[2], hi[3]);                               \
      if (HILO) {                                                                                                \
        if (with_lo) *(uint4*)(Yl + yst + v * YRG * WT) = make_uint4(lo[0], lo[1], lo[2], lo[3]);                \
      }                                                                                                          \
    }                                                                                                            \
  }

    // ---- prologue: scales of the first two chunks, pieces 0 and 1 in registers, piece 0 staged, piece 2 requested
    {
      load_scales(c_first);
      const float sc0 = scale_value(c_first);
      load_scales(c_first + c_step);
      const float sc1 = scale_value(NC > 1 ? c_first + c_step : -1);
      if (tid < kChunk) {
        scl[srow] = sc0;
        scl[kChunk + srow] = sc1;
        if (do_n) {
          write_n_operand(0, sc0);
          write_n_operand(1, sc1);
        }
      }
      for (int k = tid; k < kGBlock && k < NC; k += NTP) gl[k] = a.gbar[(size_t)bh * NC + c_first + k * c_step];
    }
    load_scales(c_first + 2 * c_step);  // consumed (table write) at the last piece of the first chunk
    // (the prefetches are unconditional, past the end the last piece is fetched again: a conditional prefetch makes
    // the compiler keep the register sets in scratch memory across the loop back-edge)
    MLSTM_SCAN_PREFETCH(0, 0)
    MLSTM_SCAN_PREFETCH(1, max(min(1, total - 1), 0))
    __syncthreads();  // scale table visible
    MLSTM_SCAN_STAGE(0, 0, 0)
    MLSTM_SCAN_PREFETCH(0, max(min(2, total - 1), 0))

    // one piece p of parity PAR (its LDS buffer); the pieces p+1 and p+3 use the other buffer and register set
#define MLSTM_SCAN_BODY(PAR, OTHER, p_)                                                                          \
  {                                                                                                              \
    const int it = (p_) / NP, piece = (p_) % NP;                                                                 \
    const int c = c_first + it * c_step;                                                                         \
    /* The decay factors come from LDS, a block of chunks at a time. */                                          \
    if (refill_due(p_)) {                                                                                        \
      __syncthreads();                                                                                           \
      for (int k = tid; k < kGBlock && it + k < NC; k += NTP) gl[k] = a.gbar[(size_t)bh * NC + c + k * c_step];  \
    }                                                                                                            \
    /* piece p staged; the consumers are done with piece p-1, whose buffer is staged into next */                \
    __syncthreads();                                                                                             \
    if (piece == NP - 1) {                                                                                       \
      /* Table entry of chunk it+2 (its factors were fetched one chunk ago) into the slot of chunk it, all of */ \
      /* whose pieces have been staged; it is read from the next piece on.  Then the factors of chunk it+3 are */\
      /* requested, first in this piece's batch of loads. */                                                     \
      if (tid < kChunk) {                                                                                        \
        const float sn = scale_value(it + 2 < NC ? c + 2 * c_step : -1);                                         \
        scl[(it & 1) * kChunk + srow] = sn;                                                                      \
        if (do_n) write_n_operand(it + 2, sn);                                                                   \
      }                                                                                                          \
      load_scales(c + 3 * c_step);                                                                               \
    }                                                                                                            \
    if ((p_) + 1 < total) MLSTM_SCAN_STAGE(OTHER, (p_) + 1, OTHER)                                               \
    MLSTM_SCAN_PREFETCH(OTHER, min((p_) + 3, total - 1))                                                         \
  }
    for (int p = 0; p < total; p += 2) {
      MLSTM_SCAN_BODY(0, 1, p)
      if (p + 1 < total) MLSTM_SCAN_BODY(1, 0, p + 1)
    }
#undef MLSTM_SCAN_BODY
#undef MLSTM_SCAN_STAGE
#undef MLSTM_SCAN_PREFETCH
  } else {
    // ======================================================================================= consumer waves
    // the normaliser vector rides with two waves of every 64 state rows in the first column tile: value-column blocks
    // 0 and 1 carry it for the first and the second 32 rows
    const bool with_n = (a.nstates != nullptr) && blk.y == 0;
    if (with_n && wave % WC == 0)
      scan_consumer<RT, WT, F16, 0>(a, bufs, gl, nB, wave, lane, bh, d_tile, w_tile, n_run);
    else if (with_n && wave % WC == 1)
      scan_consumer<RT, WT, F16, 1>(a, bufs, gl, nB, wave, lane, bh, d_tile, w_tile, n_run);
    else
      scan_consumer<RT, WT, F16, -1>(a, bufs, gl, nB, wave, lane, bh, d_tile, w_tile, n_run);
  }
}

template <int RT, int WT, bool F16>
static const char* launch_scan_roles_f(const ScanArgs& a, int BH, hipStream_t stream) {
  constexpr int NW = (RT / 64) * (WT / 32);
  const size_t smem = (size_t)2 * kChunk * (RT + WT) * 2 + (size_t)(kGBlock + 2 * kChunk) * 4 + (size_t)3 * kChunk * 3 * 2;
  if (hipFuncSetAttribute((const void*)scan_roles_kernel<RT, WT, F16>, hipFuncAttributeMaxDynamicSharedMemorySize,
                          (int)smem) != hipSuccess)
    return "scan: cannot raise the dynamic LDS limit";
  dim3 grid(a.DHQK / RT, a.DHHV / WT, BH);
  hipLaunchKernelGGL((scan_roles_kernel<RT, WT, F16>), grid, dim3(128 * NW), smem, stream, a);
  return nullptr;
}
template <int RT, int WT>
static const char* launch_scan_roles_t(const ScanArgs& a, int BH, hipStream_t stream) {
  return a.f16 ? launch_scan_roles_f<RT, WT, true>(a, BH, stream) : launch_scan_roles_f<RT, WT, false>(a, BH, stream);
}

const char* launch_scan(const ScanArgs& a_in, int BH, bool hilo, hipStream_t stream) {
  ScanArgs a = a_in;
  a.part = 0;
  if (a.DHQK % 64 != 0 || a.DHHV % 64 != 0) return "scan: DHQK and DHHV must be multiples of 64";
  if (a.stride < 1 || a.stride > kMaxStateStride) return "scan: state stride out of range";
  const bool r128 = a.DHQK % 128 == 0, w128 = a.DHHV % 128 == 0;
  auto roles = [&]() -> const char* {
    if (r128 && w128) return launch_scan_roles_t<128, 128>(a, BH, stream);
    if (r128) return launch_scan_roles_t<128, 64>(a, BH, stream);
    if (w128) return launch_scan_roles_t<64, 128>(a, BH, stream);
    return launch_scan_roles_t<64, 64>(a, BH, stream);
  };
  if (hilo) {
    // Two launches (forward only): the chunks whose rounding no longer shows in the last state go through the faster
    // kernel without the remainder operand, which leaves its state in final_out / n_final; the kernel with the
    // remainder continues from there.  Both find the chunk where they meet from the decay factors alone.
    if (a.final_out == nullptr || a.backward) return "scan: the remainder split serves the forward last state only";
    const bool two = a.nstates == nullptr || a.n_final != nullptr;  // n needs its hand-over buffer too
    if (two) {
      a.part = 1;
      if (const char* e = roles()) return e;
      a.part = 2;
    }
    if (r128 && w128) return launch_scan_t<128, 128, true>(a, BH, stream);
    if (r128) return launch_scan_t<128, 64, true>(a, BH, stream);
    if (w128) return launch_scan_t<64, 128, true>(a, BH, stream);
    return launch_scan_t<64, 64, true>(a, BH, stream);
  }
  return roles();
}

}  // namespace mlstm
