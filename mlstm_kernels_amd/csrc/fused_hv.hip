// Sequential fused kernels of the chunkwise mLSTM whose output tile spans value columns: the forward pass
// (state recurrence + output H) and the backward pass for dV (dC recurrence + dV), one launch each.
//
//   forward, chunk c = 0 .. NC-1   (mlstm_kernels/torch/chunkwise/native/fw.py:88-212 in the reference):
//     H_c   = [ bbar/sqrt(d) . (Q_c C_{c-1})  +  Sbar_c V_c ] / (max(|den|, floor) + eps)
//     C_c   = gbar_c C_{c-1} + K_c^T (abar . V_c)                  n_c likewise
//   backward, chunk c = NC-1 .. 0  (mlstm_kernels/torch/chunkwise/native/bw.py:67-198):
//     dV_c     = Sbar_c^T (rho . dH_c)  +  abar . (K_c dC_c)
//     dC_{c-1} = gbar_c dC_c + Q_c^T (rho . bbar/sqrt(d) . dH_c)
//
// A workgroup owns one (batch, head) pair and a slice of 64 value columns and walks the chunks in order.  Its
// (DHQK x 64) fp32 state slice lives in MFMA accumulators for the whole sequence and never goes to HBM unless the
// caller asks for the per-chunk states (the dQ/dK kernels of a later backward pass consume them); K, V (or Q, dH)
// are read once per slice from L2 -- the slices of one head run on the same XCD -- and once from HBM.  Compared
// with a separate state scan followed by a chunk-parallel output kernel this removes one write and one read of
// every chunk state (2 x DHQK x DHHV x 2 B per chunk and head) and one pass over the inputs.
//
// Roles (n = position index of the output rows, o = the other position index of the score matrix):
//   forward: Xn = Q (n = t), Xo = K (o = j <= t), Xw = V,  update scale = abar_j
//   dV     : Xn = K (n = j), Xo = Q (o = t >= j), Xw = dH, update scale = bbar_t/sqrt(d) * rho_t
// Per chunk, with two barriers (the waves run independently in between; wave = one 32-position block of the
// output rows and one quarter of the state rows):
//   staging   registers -> LDS: Xo rows, Xw rows (raw, and scaled for the update, split hi/lo in the forward), gate
//             vectors; the state slice is rounded to bf16 and laid out as A-operand fragments in LDS (and HBM on
//             request).  Barrier.
//   inter     Out^T[w][n] = State^T[w][d] Xn^T[d][n], Xn fragments straight from global memory in registers
//   scores    per live 32x32 block: S^T[o][n] = Xo Xn^T, gated in fp32 in the accumulator registers, rounded, and
//             used at once as the B operand of  Out^T += Xw^T P  (the transposing read enumerates the value rows in
//             accumulator order); the score matrix never touches LDS.  Row sums and q . n_prev give the denominators.
//   update    state <- gbar * state + Xo^T (scale . Xw); the next chunk's rows are requested just before
//   store     output rows (normalised), Xn fragments of the next chunk requested.  Barrier.
// All LDS tiles are unpadded and XOR-swizzled at 16-byte granularity (row-fragment reads, transposing reads and
// staging writes are conflict-free), which is what lets the 64 KB Xo tile, three value tiles and the state
// fragments share the 160 KB of one CU.
//
// Status: correct on every tested shape, but latency-bound.  With one four-wave workgroup per CU (the LDS footprint
// allows no second one) each SIMD runs a single instruction stream, so LDS latency, vector work and matrix work
// add up instead of overlapping: 26k cycles per chunk against 5k of matrix-pipe time.  Measured at B=4, S=16384,
// NH=8, 256/512 on MI355X: forward 1.56 ms, dV 1.28 ms, at a third of the HBM traffic of the split form, whose scan
// plus streaming kernel take about half that time.  The host therefore selects these kernels only on request.
#include "common.h"
#include "kernels.h"

namespace mlstm {

namespace {
// 16-byte-unit swizzle of a tile row: 4 consecutive rows map to 4 distinct 32-byte slots (transposing reads),
// 8 consecutive rows to 8 distinct 16-byte slots (row-fragment reads)
__device__ __forceinline__ int sw3(int row) { return ((row & 3) << 1) | ((row >> 2) & 1); }

__device__ __forceinline__ void mfma32v(f32x16& acc, const u32x4& a, const u32x4& b) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
}
// Transposing fragment read from a swizzled tile with ROWLEN elements per row.  A fragment covers rows
// k0 .. k0+15 (contraction index, k0 a multiple of 16) and columns col0 .. col0+31.  The swizzle of the rows a lane
// touches does not depend on k0, so the two per-lane element offsets are computed once (TrOff) and every
// fragment of the same column block is an immediate offset away.
struct TrOff {
  int lo, hi;
};
template <int ROWLEN>
__device__ __forceinline__ TrOff tr_offsets(int col0, int lane, int row0, int row_step) {
  // row0: first of the 4 rows of this lane's half-wave in the first read; the second read is row_step rows
  // further.  (8h, 4) enumerates the 16 rows in natural order: slots 0-3 <- rows 8h..8h+3, slots 4-7 <- 8h+4..;
  // (4h, 8) enumerates them in accumulator order: slots 0-3 <- rows 4h..4h+3, slots 4-7 <- rows 8+4h..
  const int q16 = (lane >> 4) & 1, i16 = lane & 15;
  const int krow = row0 + (i16 >> 2);
  const int col = col0 + 16 * q16 + 4 * (i16 & 3);
  const int unit = col >> 3, sub = col & 7;
  TrOff o;
  o.lo = krow * ROWLEN + ((unit ^ sw3(krow)) << 3) + sub;
  o.hi = (krow + row_step) * ROWLEN + ((unit ^ sw3(krow + row_step)) << 3) + sub;
  return o;
}
template <int ROWLEN>
__device__ __forceinline__ u32x4 tr_frag(const uint16_t* tile, int k0, const TrOff& o) {
  const uint2 lo = lds_read_tr16(tile + k0 * ROWLEN + o.lo);
  const uint2 hi = lds_read_tr16(tile + k0 * ROWLEN + o.hi);
  u32x4 f = {lo.x, lo.y, hi.x, hi.y};
  return f;
}
}  // namespace

// NWQ = waves per 32-position block: 1 (four waves, one per SIMD, each with the whole register file and both
// 32-column value blocks) or 2 (eight waves, two per SIMD: the pair shares the position block, each wave takes
// one value block and both compute the block's scores -- redundant matrix work bought for a second instruction
// stream per SIMD that fills the other one's stalls).
template <int DQ, bool IS_DV, bool HILO, int NWQ>
__global__ __launch_bounds__(256 * NWQ) __attribute__((amdgpu_waves_per_eu(NWQ, NWQ))) void fused_hv_kernel(FusedHvArgs a) {
  constexpr int NTH = 256 * NWQ;
  constexpr int NW = 4 * NWQ;         // waves
  constexpr int WPW = 2 / NWQ;        // 32-column value blocks per wave
  constexpr int ND = DQ / 16;         // contraction steps over the head dimension
  constexpr int DBW = DQ / 128;       // 32-row state blocks per wave (times its value blocks)
  constexpr int KU = DQ / 8;          // 16-byte units per Xo row
  constexpr int KV = 128 * KU / NTH;  // Xo units per thread per chunk
  constexpr int VV = 128 * 8 / NTH;   // Xw units per thread per chunk
  constexpr int NK = (DQ + NTH - 1) / NTH;
  constexpr int SB = NWQ == 1 ? 8 : 4;  // row fragments fetched ahead of the matrix instructions that use them
  extern __shared__ __align__(16) unsigned char smem_raw[];
  uint16_t* Ks = (uint16_t*)smem_raw;  // [128][DQ]   Xo rows of the chunk
  uint16_t* Vr = Ks + 128 * DQ;        // [128][64]   Xw rows, raw
  uint16_t* Vh = Vr + 128 * 64;        // [128][64]   scaled Xw rows (bf16 head)
  uint16_t* Vl = Vh + 128 * 64;        // [128][64]   bf16 remainder of the scaled rows (forward)
  uint16_t* St = Vl + 128 * 64;        // state fragments [2][ND][64 lanes][8]
  float* npart = (float*)(St + 2 * ND * 512);  // [NW waves][DQ] partial sums of the n update
  float* ua = npart + NW * DQ;         // [2][128] update scale per position, double-buffered by chunk parity
  float* uu = ua + 256;                // [128] u_t
  float* ww = uu + 128;                // [128] w_j
  float* cs = ww + 128;                // [128] column scale of the inter-chunk product
  float* gxs = cs + 128;               // [128] forward: mcomb_t; dV: rho_t
  float* nv = gxs + 128;               // [2][DQ] normaliser state n, double-buffered by chunk parity
  float* gdl = nv + 2 * DQ;            // [2] decay factor gbar of the chunk, double-buffered by chunk parity

  // the wave index is made scalar so that branches on it are scalar branches
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, h = lane >> 5;
  const int nb = wave & 3;   // 32-position block of the output rows, and group of state rows, handled by this wave
  const int wq = wave >> 2;  // which of the NWQ waves of that block: owns value blocks wq * WPW .. + WPW - 1
  const BlockId blk = xcd_block_id();  // the slices of one (batch, head) get consecutive ids: same XCD, shared L2
  const int bh = blk.y;
  const int w_tile = blk.x * 64;
  const int DHHV = a.DHHV, S = a.S, NC = a.NC;
  const size_t Sp = (size_t)NC * kChunk;
  const bool do_n = !IS_DV && a.use_nrow;
  const char* Xn_g = (const char*)((IS_DV ? a.K : a.Q) + (size_t)bh * S * DQ);
  const char* Xo_g = (const char*)((IS_DV ? a.Q : a.K) + (size_t)bh * S * DQ);
  const char* Xw_g = (const char*)((IS_DV ? a.dH : a.V) + (size_t)bh * S * DHHV + w_tile);
  const float* usc_g = (IS_DV ? a.g.bbar : a.g.abar) + bh * Sp;  // update scale per position
  const float* csc_g = (IS_DV ? a.g.abar : a.g.bbar) + bh * Sp;  // column scale per position
  // dV: row normaliser of the forward pass (any valid vector when the variant is un-normalised: it is ignored)
  const float* nr_g = (IS_DV && a.use_nrow) ? a.nrow + bh * Sp : usc_g;

  // ---- state slice: wave owns state rows 32 * (nb * DBW + db) .. +31, all 64 value columns
  f32x16 acc[DBW][WPW];
#pragma unroll
  for (int db = 0; db < DBW; ++db)
#pragma unroll
    for (int wb = 0; wb < WPW; ++wb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[db][wb][i] = 0.f;
  if (a.init != nullptr) {
    const float* src = a.init + ((size_t)bh * DQ + 32 * nb * DBW + 4 * h) * DHHV + w_tile + 32 * wq * WPW + r;
#pragma unroll
    for (int db = 0; db < DBW; ++db)
#pragma unroll
      for (int wb = 0; wb < WPW; ++wb)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[db][wb][i] = src[(size_t)(32 * db + 8 * (i / 4) + (i % 4)) * DHHV + 32 * wb];
  }
  for (int d = tid; d < DQ; d += NTH) nv[d] = (do_n && a.n_init != nullptr) ? a.n_init[(size_t)bh * DQ + d] : 0.f;

  u32x4 kreg[KV], vreg[VV], qf[ND];
  float gu = 0.f, gw = 0.f, gcs = 0.f, gx = 0.f, gus = 0.f, ggd = 0.f;
  // Loads only: no arithmetic touches a prefetched register before its consumer phase (an early use would make
  // the wave wait for the whole batch).  Macros, so that the register arrays are never captured by reference.
  // Rows past the end of the sequence are read from the last valid row instead of being zeroed (no branch, no
  // select on a loaded value): their update scale is 0, their score entries are masked, their output rows are
  // not stored.  Offsets inside one (batch, head) fit 32 bits (checked by the launcher).
#define MLSTM_PREFETCH_KV(c_)                                                                                 \
  {                                                                                                           \
    const int tb_ = (c_) * kChunk;                                                                            \
    if (tb_ + kChunk <= S) {                                                                                  \
      /* whole chunk inside the sequence: uniform base + one per-lane offset + constants */                   \
      const char* kb_ = Xo_g + (size_t)tb_ * (DQ * 2);                                                        \
      const char* vb_ = Xw_g + (size_t)tb_ * DHHV * 2;                                                        \
      _Pragma("unroll") for (int v = 0; v < KV; ++v)                                                          \
          kreg[v] = *(const u32x4*)(kb_ + v * (NTH / KU) * (DQ * 2) + klane);                                 \
      _Pragma("unroll") for (int v = 0; v < VV; ++v)                                                          \
          vreg[v] = *(const u32x4*)(vb_ + (size_t)v * (NTH / 8) * DHHV * 2 + vlane);                          \
    } else {                                                                                                  \
      /* ragged last chunk; the opaque copy of the thread index keeps these row computations out of the */    \
      /* registers that live across the chunk loop */                                                         \
      int tv_ = tid;                                                                                          \
      asm volatile("" : "+v"(tv_));                                                                           \
      _Pragma("unroll") for (int v = 0; v < KV; ++v) {                                                        \
        const int idx = tv_ + v * NTH;                                                                        \
        const uint32_t row = (uint32_t)min(tb_ + idx / KU, S - 1);                                            \
        kreg[v] = *(const u32x4*)(Xo_g + (row * (uint32_t)(DQ * 2) + (uint32_t)((idx % KU) * 16)));           \
      }                                                                                                       \
      _Pragma("unroll") for (int v = 0; v < VV; ++v) {                                                        \
        const int idx = tv_ + v * NTH;                                                                        \
        const uint32_t row = (uint32_t)min(tb_ + (idx >> 3), S - 1);                                          \
        vreg[v] = *(const u32x4*)(Xw_g + (row * (uint32_t)(DHHV * 2) + (uint32_t)((idx & 7) * 16)));          \
      }                                                                                                       \
    }                                                                                                         \
  }
#define MLSTM_PREFETCH_GATES(c_)                                                                              \
  if (tid < 128) {                                                                                            \
    const int tb_ = (c_) * kChunk;                                                                            \
    gu = a.g.u[bh * Sp + tb_ + tid];                                                                          \
    gw = a.g.w[bh * Sp + tb_ + tid];                                                                          \
    gcs = csc_g[tb_ + tid];                                                                                   \
    gx = IS_DV ? nr_g[tb_ + tid] : a.g.mcomb[bh * Sp + tb_ + tid];                                            \
    gus = usc_g[min(tb_ + tid, S - 1)];                                                                       \
    ggd = a.g.gbar[(size_t)bh * NC + (c_)];                                                                   \
  }
#define MLSTM_LOAD_XN(c_)                                                                                     \
  {                                                                                                           \
    const uint32_t row = (uint32_t)min((c_) * kChunk + 32 * nb + r, S - 1);                                   \
    const u32x4* src = (const u32x4*)(Xn_g + (row * (uint32_t)(DQ * 2) + (uint32_t)(16 * h)));                \
    _Pragma("unroll") for (int ds = 0; ds < ND; ++ds) qf[ds] = src[2 * ds];                                   \
  }
  // update scale of the prefetched chunk -> LDS (forward abar_j; dV bbar_t/sqrt(d)/(nrow_t + eps)); positions past
  // the end of the sequence get 0 and so neither feed the state nor the normaliser
#define MLSTM_PUBLISH_SCALE(buf_, c_)                                                                         \
  if (tid < 128) {                                                                                            \
    const float us_ = (c_) * kChunk + tid < S ? gus : 0.f;                                                    \
    ua[(buf_) * 128 + tid] = IS_DV ? us_ * a.qk_scale / (a.use_nrow ? gx + a.eps : 1.f) : us_;                \
    if (tid == 0) gdl[buf_] = ggd;                                                                            \
  }

  // per-lane parts of the staging addresses: thread (row group, 16-byte unit) of the Xo and Xw tiles; the rows a
  // thread handles are 8 * k (Xo) or 32 * k (Xw) apart, so they all share the swizzle of the first one
  const uint32_t klane = (uint32_t)((tid / KU) * (DQ * 2) + (tid % KU) * 16);
  const uint32_t vlane = (uint32_t)((tid >> 3) * DHHV * 2 + (tid & 7) * 16);
  uint16_t* const kst = Ks + (tid / KU) * DQ + (((tid % KU) ^ sw3(tid / KU)) << 3);
  const int vst = (tid >> 3) * 64 + (((tid & 7) ^ sw3(tid >> 3)) << 3);
  static_assert((NTH / KU) % 8 == 0 && (NTH / 8) % 8 == 0, "row groups must preserve the swizzle");

  const int c_first = IS_DV ? NC - 1 : 0, c_step = IS_DV ? -1 : 1;
  MLSTM_PREFETCH_GATES(c_first);
  MLSTM_PREFETCH_KV(c_first);
  MLSTM_LOAD_XN(c_first);
  MLSTM_PUBLISH_SCALE(0, c_first);
  __syncthreads();
  // per-lane offsets of the transposing reads: value tiles (the two 32-column blocks) in natural order of the
  // contraction index (state update) and in accumulator order (intra-chunk product, see below); Xo tile (this
  // wave's state rows)
  TrOff offV[WPW], offVp[WPW], offK[DBW];
#pragma unroll
  for (int wb = 0; wb < WPW; ++wb) {
    offV[wb] = tr_offsets<64>(32 * (wq * WPW + wb), lane, 8 * h, 4);
    offVp[wb] = tr_offsets<64>(32 * (wq * WPW + wb), lane, 4 * h, 8);
  }
#pragma unroll
  for (int db = 0; db < DBW; ++db) offK[db] = tr_offsets<DQ>(32 * (nb * DBW + db), lane, 8 * h, 4);
  // row r of every 32-row block of the Xo tile has the same swizzle: four per-lane unit offsets cover all
  // contraction steps of a row-fragment read
  int soff[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) soff[k] = ((2 * k + h) ^ sw3(r)) << 3;

  // live score blocks of this wave's output block nb: forward o-blocks 0..nb, dV o-blocks nb..3
  const int ob_lo = IS_DV ? nb : 0, ob_hi = IS_DV ? 4 : nb + 1;
  const int n = 32 * nb + r;  // position inside the chunk of this lane's output row / score column
  constexpr float kLog2e = 1.4426950408889634f;
  const float log2_qk = __log2f(a.qk_scale);
  for (int it = 0; it < NC; ++it) {
    const int c = c_first + it * c_step;
    const int t_base = c * kChunk;
    const bool more = it + 1 < NC;
    const float* uac = ua + (it & 1) * 128;
    const float* nvc = nv + (it & 1) * DQ;
    float* nvn = nv + ((it + 1) & 1) * DQ;
    // =========================== staging: registers -> LDS ===========================
    {
      // all per-row scales first: one round trip to LDS instead of one per row
      float scK[KV], scV[VV];
      if (do_n) {
#pragma unroll
        for (int v = 0; v < KV; ++v) scK[v] = uac[tid / KU + v * (NTH / KU)];
      }
#pragma unroll
      for (int v = 0; v < VV; ++v) scV[v] = uac[(tid >> 3) + v * (NTH / 8)];
      float np[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int v = 0; v < KV; ++v) {
        *(u32x4*)(kst + v * (NTH / KU) * DQ) = kreg[v];
        if (do_n) {
          const float xs = scK[v];
#pragma unroll
          for (int p = 0; p < 4; ++p) {
            np[2 * p] += xs * __uint_as_float(kreg[v][p] << 16);
            np[2 * p + 1] += xs * __uint_as_float(kreg[v][p] & 0xffff0000u);
          }
        }
      }
      if (do_n) {
        // a wave covers 64 / KU row groups of all KU column units: fold them, one partial row per wave
#pragma unroll
        for (int o = 32; o >= KU; o >>= 1)
#pragma unroll
          for (int p = 0; p < 8; ++p) np[p] += __shfl_xor(np[p], o);
        if (lane < KU) {
          float* dst = npart + wave * DQ + lane * 8;
          *(float4*)dst = make_float4(np[0], np[1], np[2], np[3]);
          *(float4*)(dst + 4) = make_float4(np[4], np[5], np[6], np[7]);
        }
      }
#pragma unroll
      for (int v = 0; v < VV; ++v) {
        const int o = vst + v * (NTH / 8) * 64;
        const float sc = scV[v];
        u32x4 hi, lo;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          const float e0 = __uint_as_float(vreg[v][p] << 16) * sc;
          const float e1 = __uint_as_float(vreg[v][p] & 0xffff0000u) * sc;
          hi[p] = pack_bf16x2(e0, e1);
          if (HILO) lo[p] = pack_bf16x2(e0 - __uint_as_float(hi[p] << 16), e1 - __uint_as_float(hi[p] & 0xffff0000u));
        }
        *(u32x4*)(Vr + o) = vreg[v];
        *(u32x4*)(Vh + o) = hi;
        if (HILO) *(u32x4*)(Vl + o) = lo;
      }
      if (tid < 128) {
        // exponents in base 2 (one v_exp_f32 per score); the 1/sqrt(d) of the scores rides in u (forward) / w (dV)
        uu[tid] = gu * kLog2e + (IS_DV ? 0.f : log2_qk);
        ww[tid] = gw * kLog2e - (IS_DV ? log2_qk : 0.f);
        cs[tid] = IS_DV ? gcs : gcs * a.qk_scale;
        gxs[tid] = IS_DV ? (a.use_nrow ? 1.f / (gx + a.eps) : 1.f) : gx;
      }
      // state before this chunk's update -> bf16 fragments: LDS (natural order of the contraction index, so that
      // Xn fragments are plain 16-byte loads of a row) and, on request, HBM (the stored fragment format)
      // kept boundaries only: forward the state before every stride-th chunk, dV the gradient of the state after the
      // last chunk of every group of `stride` chunks (and after the last chunk of the sequence); slot c / stride
      const bool keep_state = IS_DV ? (c == NC - 1 || (c + 1) % a.stride == 0) : (c % a.stride == 0);
      const size_t NCS = (size_t)(NC + a.stride - 1) / a.stride;
      u32x4* stg = (a.states == nullptr || !keep_state)
                       ? nullptr
                       : (u32x4*)a.states + ((size_t)bh * NCS + c / a.stride) * (size_t)(DHHV / 32) * ND * 64;
#pragma unroll
      for (int db = 0; db < DBW; ++db)
#pragma unroll
        for (int wk = 0; wk < WPW; ++wk)
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const int wb = wq * WPW + wk;
            u32x4 f;
            f[0] = pack_bf16x2(acc[db][wk][8 * half + 0], acc[db][wk][8 * half + 1]);
            f[1] = pack_bf16x2(acc[db][wk][8 * half + 2], acc[db][wk][8 * half + 3]);
            f[2] = pack_bf16x2(acc[db][wk][8 * half + 4], acc[db][wk][8 * half + 5]);
            f[3] = pack_bf16x2(acc[db][wk][8 * half + 6], acc[db][wk][8 * half + 7]);
            const int D16 = 2 * (nb * DBW + db) + half;
            uint16_t* frag = St + (size_t)(wb * ND + D16) * 512;
            *(uint2*)(frag + r * 8 + 4 * h) = make_uint2(f[0], f[1]);
            *(uint2*)(frag + (32 + r) * 8 + 4 * h) = make_uint2(f[2], f[3]);
            if (stg != nullptr) stg[((size_t)((w_tile >> 5) + wb) * ND + D16) * 64 + lane] = f;
          }
    }
    __syncthreads();  // ---- everything staged for this chunk is visible; from here on the waves run independently
    const float gdec = gdl[it & 1];  // decay of this chunk (through LDS: no dependence on loads in flight)

    // =========================== inter-chunk product ===========================
    if (more) MLSTM_PREFETCH_GATES(c + c_step);  // consumed at the end of this iteration
    float nsum[NK];
    if (do_n) {
#pragma unroll
      for (int k = 0; k < NK; ++k) {
        const int d = tid + k * NTH;
        float sm = 0.f;
        if (d < DQ) {
#pragma unroll
          for (int w4 = 0; w4 < NW; ++w4) sm += npart[w4 * DQ + d];
        }
        nsum[k] = sm;
      }
    }
    f32x16 oacc[WPW];
#pragma unroll
    for (int wb = 0; wb < WPW; ++wb)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[wb][i] = 0.f;
    {
      const u32x4* sf = (const u32x4*)St + (size_t)wq * WPW * ND * 64 + lane;
#pragma unroll
      for (int d0 = 0; d0 < ND; d0 += 4) {
        u32x4 A[WPW][4];
#pragma unroll
        for (int k = 0; k < 4; ++k)
#pragma unroll
          for (int wb = 0; wb < WPW; ++wb) A[wb][k] = sf[(wb * ND + d0 + k) * 64];
#pragma unroll
        for (int k = 0; k < 4; ++k)
#pragma unroll
          for (int wb = 0; wb < WPW; ++wb) mfma32v(oacc[wb], A[wb][k], qf[d0 + k]);
      }
    }
    const float csn = cs[n];
#pragma unroll
    for (int wb = 0; wb < WPW; ++wb) oacc[wb] *= csn;

    // =========================== score blocks, gated in registers, times the value rows ===========================
    // A gated 32x32 score block never leaves the wave: in accumulator layout lane (r, h) holds, for its column n,
    // the rows o = 8g + 4h + e, and exactly these eight values per 16 rows form a B operand if the contraction
    // index is enumerated in that order -- which the transposing read of the value rows can do (offVp).
    float rsum = 0.f;
    {
      const float un = IS_DV ? ww[n] : uu[n];
      const int valid = S - t_base;  // positions of this chunk inside the sequence
      for (int ob = ob_lo; ob < ob_hi; ++ob) {
        f32x16 sacc;
#pragma unroll
        for (int i = 0; i < 16; ++i) sacc[i] = 0.f;
        const uint16_t* krow_p = Ks + (32 * ob + r) * DQ;
        // gate vectors of the block's 32 rows, fetched before the matrix instructions so that their latency is covered
        float4 xo4[4], rr4[4];
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          xo4[g4] = *(const float4*)((IS_DV ? uu : ww) + 32 * ob + 8 * g4 + 4 * h);
          if (IS_DV) rr4[g4] = *(const float4*)(gxs + 32 * ob + 8 * g4 + 4 * h);
        }
#pragma unroll
        for (int d0 = 0; d0 < ND; d0 += SB) {
          u32x4 A[SB];
#pragma unroll
          for (int k = 0; k < SB; ++k) A[k] = *(const u32x4*)(krow_p + ((d0 + k) >> 2) * 64 + soff[(d0 + k) & 3]);
#pragma unroll
          for (int k = 0; k < SB; ++k) mfma32v(sacc, A[k], qf[d0 + k]);
        }
        u32x4 Bp[2];
        float pv[16];
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const float4 xo = xo4[g4];
          const float xov[4] = {xo.x, xo.y, xo.z, xo.w};
          float rho[4] = {1.f, 1.f, 1.f, 1.f};
          if (IS_DV) {
            const float4 rr = rr4[g4];
            rho[0] = rr.x; rho[1] = rr.y; rho[2] = rr.z; rho[3] = rr.w;
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float ex = IS_DV ? (xov[e] - un) : (un - xov[e]);   // (u_t - w_j) log2(e) + log2(1/sqrt(d))
            float val = sacc[4 * g4 + e] * __builtin_amdgcn_exp2f(ex);
            if (IS_DV) val *= rho[e];
            pv[4 * g4 + e] = val;
          }
        }
        // masks: causal (only the diagonal block has masked entries) and end of sequence (only the last chunk)
        if (ob == nb || valid < kChunk) {
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int o = 32 * ob + 8 * (i / 4) + 4 * h + (i % 4);
            const bool keep = (IS_DV ? (n <= o) : (o <= n)) && (o < valid);
            pv[i] = keep ? pv[i] : 0.f;
          }
        }
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          if (!IS_DV) rsum += pv[i] + pv[i + 1];
          Bp[i >> 3][(i >> 1) & 3] = pack_bf16x2(pv[i], pv[i + 1]);
        }
#pragma unroll
        for (int jl = 0; jl < 2; ++jl)
#pragma unroll
          for (int wb = 0; wb < WPW; ++wb) {
            const u32x4 A = tr_frag<64>(Vr, 32 * ob + 16 * jl, offVp[wb]);
            mfma32v(oacc[wb], A, Bp[jl]);
          }
      }
    }
    // ---- denominators (forward): every lane owns the row sums and q.n of its position
    float iv = 1.f;
    if (!IS_DV) {
      float nmax = 1.f;
      if (a.use_nrow) {
        float dot = 0.f;
#pragma unroll
        for (int ds = 0; ds < ND; ++ds) {
          const float4 n0 = *(const float4*)(nvc + 16 * ds + 8 * h);
          const float4 n1 = *(const float4*)(nvc + 16 * ds + 8 * h + 4);
          const float nn[8] = {n0.x, n0.y, n0.z, n0.w, n1.x, n1.y, n1.z, n1.w};
#pragma unroll
          for (int p = 0; p < 4; ++p) {
            dot += __uint_as_float(qf[ds][p] << 16) * nn[2 * p];
            dot += __uint_as_float(qf[ds][p] & 0xffff0000u) * nn[2 * p + 1];
          }
        }
        dot += __shfl_xor(dot, 32);
        rsum += __shfl_xor(rsum, 32);
        const float den = csn * dot + rsum;
        const float floor_v = a.sig_gate ? 1.f : __expf(-gxs[n]);
        nmax = fmaxf(fabsf(den), floor_v);
        iv = 1.f / (nmax + a.eps);
      }
      if (w_tile == 0 && h == 0 && wq == 0) {
        a.nrow_out[bh * Sp + t_base + n] = nmax;
        const int tg = t_base + n;
        if (tg < S) {
          if (a.n_out != nullptr) a.n_out[(size_t)bh * S + tg] = nmax;
          if (a.m_out != nullptr) a.m_out[(size_t)bh * S + tg] = gxs[n];
        }
      }
    }

    // =========================== state update ===========================
#pragma unroll
    for (int db = 0; db < DBW; ++db)
#pragma unroll
      for (int wb = 0; wb < WPW; ++wb) acc[db][wb] *= gdec;
    // The next chunk's rows are requested only now: loads complete in order and the wait counter cannot tell them
    // apart, so every consumer of an older load (the Xn fragments above, the decay factor) must come first.
    if (more) MLSTM_PREFETCH_KV(c + c_step);
#pragma unroll
    for (int js = 0; js < 8; ++js) {
      u32x4 A[DBW], Bh[WPW];
#pragma unroll
      for (int db = 0; db < DBW; ++db) A[db] = tr_frag<DQ>(Ks, 16 * js, offK[db]);
#pragma unroll
      for (int wb = 0; wb < WPW; ++wb) Bh[wb] = tr_frag<64>(Vh, 16 * js, offV[wb]);
#pragma unroll
      for (int db = 0; db < DBW; ++db)
#pragma unroll
        for (int wb = 0; wb < WPW; ++wb) mfma32v(acc[db][wb], A[db], Bh[wb]);
      if (HILO) {
        u32x4 Bl[WPW];
#pragma unroll
        for (int wb = 0; wb < WPW; ++wb) Bl[wb] = tr_frag<64>(Vl, 16 * js, offV[wb]);
#pragma unroll
        for (int db = 0; db < DBW; ++db)
#pragma unroll
          for (int wb = 0; wb < WPW; ++wb) mfma32v(acc[db][wb], A[db], Bl[wb]);
      }
    }
    if (do_n) {
#pragma unroll
      for (int k = 0; k < NK; ++k) {
        const int d = tid + k * NTH;
        if (d < DQ) nvn[d] = gdec * nvc[d] + nsum[k];
      }
    }

    // =========================== output rows ===========================
    {
      const int t = t_base + n;
      if (t < S) {
        uint16_t* orow = a.Out + ((size_t)bh * S + t) * DHHV + w_tile + 32 * wq * WPW + 4 * h;
#pragma unroll
        for (int wb = 0; wb < WPW; ++wb)
#pragma unroll
          for (int g4 = 0; g4 < 4; ++g4)
            *(uint2*)(orow + 32 * wb + 8 * g4) =
                make_uint2(pack_bf16x2(oacc[wb][4 * g4 + 0] * iv, oacc[wb][4 * g4 + 1] * iv),
                           pack_bf16x2(oacc[wb][4 * g4 + 2] * iv, oacc[wb][4 * g4 + 3] * iv));
      }
    }
    if (more) {
      MLSTM_LOAD_XN(c + c_step);
      MLSTM_PUBLISH_SCALE((it + 1) & 1, c + c_step);
    }
    __syncthreads();  // ---- every wave is done with this chunk's tiles
  }
#undef MLSTM_PREFETCH_KV
#undef MLSTM_PREFETCH_GATES
#undef MLSTM_LOAD_XN
#undef MLSTM_PUBLISH_SCALE

  if (a.final_out != nullptr) {
#pragma unroll
    for (int db = 0; db < DBW; ++db)
#pragma unroll
      for (int wb = 0; wb < WPW; ++wb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int d = 32 * (nb * DBW + db) + 8 * (i / 4) + 4 * h + (i % 4);
          a.final_out[((size_t)bh * DQ + d) * DHHV + w_tile + 32 * (wq * WPW + wb) + r] = acc[db][wb][i];
        }
  }
  if (do_n && a.n_final != nullptr && w_tile == 0) {
    const float* nvf = nv + (NC & 1) * DQ;
    for (int d = tid; d < DQ; d += NTH) a.n_final[(size_t)bh * DQ + d] = nvf[d];
  }
}

template <int DQ, bool IS_DV, bool HILO, int NWQ>
static const char* launch_fused_hv_t(const FusedHvArgs& a, int BH, hipStream_t stream) {
  constexpr int ND = DQ / 16;
  const size_t smem = (size_t)(128 * DQ + 3 * 128 * 64 + 2 * ND * 512) * 2 + (size_t)((2 + 4 * NWQ) * DQ + 768 + 4) * 4;
  if ((size_t)a.S * (size_t)(a.DHHV > DQ ? a.DHHV : DQ) * 2 >= ((size_t)1 << 32))
    return "fused_hv: one (batch, head) slab of an input exceeds 4 GiB";
  if (hipFuncSetAttribute((const void*)fused_hv_kernel<DQ, IS_DV, HILO, NWQ>, hipFuncAttributeMaxDynamicSharedMemorySize,
                          (int)smem) != hipSuccess)
    return "fused_hv: cannot raise the dynamic LDS limit";
  dim3 grid(a.DHHV / 64, BH);
  hipLaunchKernelGGL((fused_hv_kernel<DQ, IS_DV, HILO, NWQ>), grid, dim3(256 * NWQ), smem, stream, a);
  return nullptr;
}

bool fused_hv_supported(int DHQK, int DHHV) { return (DHQK == 128 || DHQK == 256) && DHHV % 64 == 0; }

const char* launch_fused_hv(const FusedHvArgs& a, int BH, bool is_dv, hipStream_t stream) {
  if (!fused_hv_supported(a.DHQK, a.DHHV)) return "fused_hv: unsupported head dimensions";
  if (a.stride < 1 || a.stride > kMaxStateStride) return "fused_hv: state stride out of range";
  // one wave per 32-position block (four waves, one per SIMD): the eight-wave form, in which the two waves of a block
  // both compute its scores, was measured slower
  constexpr int kWavesPerBlock = 1;
  if (is_dv) {
    if (a.DHQK == 256) return launch_fused_hv_t<256, true, false, kWavesPerBlock>(a, BH, stream);
    return launch_fused_hv_t<128, true, false, kWavesPerBlock>(a, BH, stream);
  }
  // the bf16 head + remainder split of the value operand serves the fp32 last state only
  if (a.final_out == nullptr) {
    if (a.DHQK == 256) return launch_fused_hv_t<256, false, false, kWavesPerBlock>(a, BH, stream);
    return launch_fused_hv_t<128, false, false, kWavesPerBlock>(a, BH, stream);
  }
  if (a.DHQK == 256) return launch_fused_hv_t<256, false, true, kWavesPerBlock>(a, BH, stream);
  return launch_fused_hv_t<128, false, true, kWavesPerBlock>(a, BH, stream);
}

}  // namespace mlstm
