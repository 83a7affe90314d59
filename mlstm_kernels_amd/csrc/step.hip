// Fused recurrent decode step of the mLSTM (exponential input gate), one token per (batch, head).
//
//   m' = max(logsig(f) + m, i)          f' = exp(logsig(f) + m - m')      i' = exp(i - m')
//   C' = f' C + i' k v^T                n' = f' n + i' k
//   h  = (q/sqrt(d))^T C' / (max(|q/sqrt(d) . n'|, exp(-m')) + eps)
//
// (math of mlstm_kernels/torch/recurrent/native_step.py:69-95 in the reference; everything in fp32.)
//
// The step is a pure stream over the state C (DHQK x DHHV per head; fp32, or bfloat16 when the caller keeps its states
// in that type): one read and one write of every element, 0.75 flop per byte at fp32, so it is laid out for HBM
// bandwidth only -- no matrix cores.  A workgroup owns (b, head, slice of COLS value columns); lanes of 16 B (four fp32
// or eight bf16 columns) cover one contiguous row segment and the TY
// row groups of the workgroup walk the DHQK rows with all loads of an unrolled batch in flight before the first
// use.  The q^T C' column sums are reduced across the row groups through LDS at the end.
#include "common.h"
#include "kernels.h"

namespace mlstm {

// One 16-byte piece of a state row: four fp32 columns, or eight columns when the state is kept in bfloat16 or float16
// (the reference's dtype_state / inference_state_dtype, mlstm_kernels/torch/recurrent/triton_step.py:33,67-69).
// SBF = state dtype code: 0 float32, 1 bfloat16, 2 float16.
template <int SBF>
struct StatePiece {
  static constexpr int N = SBF ? 8 : 4;
  float x[N];
};
template <int SBF, bool NT>
__device__ __forceinline__ StatePiece<SBF> load_piece(const void* base, size_t elem) {
  StatePiece<SBF> p;
  if constexpr (SBF != 0) {
    const u32x4* src = (const u32x4*)((const uint16_t*)base + elem);
    const u32x4 raw = NT ? __builtin_nontemporal_load(src) : *src;
#pragma unroll
    for (int e = 0; e < 4; ++e) unpack_state2(raw[e], SBF, p.x[2 * e], p.x[2 * e + 1]);
  } else {
    const f32x4* src = (const f32x4*)((const float*)base + elem);
    const f32x4 raw = NT ? __builtin_nontemporal_load(src) : *src;
#pragma unroll
    for (int e = 0; e < 4; ++e) p.x[e] = raw[e];
  }
  return p;
}
template <int SBF, bool NT>
__device__ __forceinline__ void store_piece(void* base, size_t elem, const StatePiece<SBF>& p) {
  if constexpr (SBF != 0) {
    const u32x4 raw = {pack_state2(p.x[0], p.x[1], SBF), pack_state2(p.x[2], p.x[3], SBF), pack_state2(p.x[4], p.x[5], SBF),
                       pack_state2(p.x[6], p.x[7], SBF)};
    u32x4* dst = (u32x4*)((uint16_t*)base + elem);
    if (NT) __builtin_nontemporal_store(raw, dst);
    else *dst = raw;
  } else {
    const f32x4 raw = {p.x[0], p.x[1], p.x[2], p.x[3]};
    f32x4* dst = (f32x4*)((float*)base + elem);
    if (NT) __builtin_nontemporal_store(raw, dst);
    else *dst = raw;
  }
}

template <int COLS, int TY, int UNROLL, bool NONTEMPORAL, int SBF>
__global__ __launch_bounds__((COLS / StatePiece<SBF>::N) * TY) void step_kernel(
    const void* __restrict__ q, const void* __restrict__ k, const void* __restrict__ v,
    const void* __restrict__ ig, const void* __restrict__ fg,
    const void* c_in, const void* n_in, const void* m_in,
    void* __restrict__ h, void* c_out, void* n_out, void* m_out,
    int DHQK, int DHHV, float eps, int dtype_qkv, int dtype_gates) {
  constexpr int VPL = StatePiece<SBF>::N;   // state columns per lane
  constexpr int TX = COLS / VPL;
  constexpr int NTH = TX * TY;
  constexpr int dtype_state = SBF;
  extern __shared__ float smem[];
  float* qs = smem;                 // [DHQK] q / sqrt(d)
  float* ik = smem + DHQK;          // [DHQK] i' * k
  float* red = smem + 2 * DHQK;     // [TY][COLS] partial column sums
  const int bh = blockIdx.y;
  const int col0 = blockIdx.x * COLS;
  const int tid = threadIdx.x;
  const int tx = tid % TX, ty = tid / TX;

  // Small states (the cacheable variant: few workgroups per CU, nothing else to hide the prologue behind): the
  // first batch of state rows is requested before anything else, so that the loads travel while the gates, q.n'
  // and the LDS staging below are computed (none of which they depend on).  With a large state many workgroups
  // per CU overlap each other's prologues and the extra live registers only cost occupancy (measured: 0.373 ms
  // against 0.358 ms at B = 256), so the streaming variant does not do it.
  const int col = col0 + VPL * tx;
  const bool col_ok = col < DHHV;  // DHHV % VPL == 0 is checked on the host
  const size_t cbase = (size_t)bh * DHQK * DHHV + col;
  const bool have_first = !NONTEMPORAL && col_ok && ty + (UNROLL - 1) * TY < DHQK;
  StatePiece<SBF> cfirst[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    if (have_first) {
      cfirst[u] = load_piece<SBF, false>(c_in, cbase + (size_t)(ty + u * TY) * DHHV);
    } else {
#pragma unroll
      for (int e = 0; e < VPL; ++e) cfirst[u].x[e] = 0.f;
    }
  }

  const float fpre = load_scalar(fg, bh, dtype_gates);
  const float ipre = load_scalar(ig, bh, dtype_gates);
  const float m_old = load_state_scalar(m_in, bh, dtype_state);
  const float lf = log_sigmoid(fpre);
  const float m_new = fmaxf(lf + m_old, ipre);
  const float fa = expf(lf + m_old - m_new);
  const float ia = expf(ipre - m_new);
  const float scale = rsqrtf((float)DHQK);

  // q.n' over the whole head (every workgroup needs it for the denominator)
  float qn_part = 0.f;
  for (int d = tid; d < DHQK; d += NTH) {
    const size_t o = (size_t)bh * DHQK + d;
    const float qd = load_scalar(q, o, dtype_qkv) * scale;
    const float kd = load_scalar(k, o, dtype_qkv);
    const float nd = fa * load_state_scalar(n_in, o, dtype_state) + ia * kd;
    qs[d] = qd;
    ik[d] = ia * kd;
    qn_part += qd * nd;
    if (blockIdx.x == 0) store_state_scalar(n_out, o, dtype_state, nd);
  }
  qn_part = wave_sum(qn_part);
  __shared__ float wsum[(NTH + kWave - 1) / kWave];
  if ((tid & 63) == 0) wsum[tid >> 6] = qn_part;
  __syncthreads();
  float qn = 0.f;
#pragma unroll
  for (int w = 0; w < (NTH + kWave - 1) / kWave; ++w) qn += wsum[w];
  const float inv_den = 1.f / (fmaxf(fabsf(qn), expf(-m_new)) + eps);
  if (blockIdx.x == 0 && tid == 0) store_state_scalar(m_out, bh, dtype_state, m_new);

  float vv[VPL];
#pragma unroll
  for (int e = 0; e < VPL; ++e) vv[e] = 0.f;
  if (col_ok) {
    const size_t o = (size_t)bh * DHHV + col;
    if (dtype_qkv == 0) {
#pragma unroll
      for (int e4 = 0; e4 < VPL / 4; ++e4) {
        const f32x4 raw = *(const f32x4*)((const float*)v + o + 4 * e4);
#pragma unroll
        for (int e = 0; e < 4; ++e) vv[4 * e4 + e] = raw[e];
      }
    } else {
#pragma unroll
      for (int e4 = 0; e4 < VPL / 4; ++e4) {
        const uint2 raw = *(const uint2*)((const uint16_t*)v + o + 4 * e4);
        unpack_state2(raw.x, dtype_qkv, vv[4 * e4 + 0], vv[4 * e4 + 1]);   // dtype code 1 bf16, 2 fp16
        unpack_state2(raw.y, dtype_qkv, vv[4 * e4 + 2], vv[4 * e4 + 3]);
      }
    }
  }
  float acc[VPL];
#pragma unroll
  for (int e = 0; e < VPL; ++e) acc[e] = 0.f;
  // C' = f' C + i' k v^T for one piece of row rr; q^T C' accumulates from the fp32 values (before any rounding)
  auto update = [&](const StatePiece<SBF>& cold, int rr) {
    StatePiece<SBF> o;
    const float ikr = ik[rr], qr = qs[rr];
#pragma unroll
    for (int e = 0; e < VPL; ++e) {
      o.x[e] = fa * cold.x[e] + ikr * vv[e];
      acc[e] += qr * o.x[e];
    }
    return o;
  };
  if (col_ok) {
    int r = ty;
    if (have_first) {
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int rr = r + u * TY;
        store_piece<SBF, false>(c_out, cbase + (size_t)rr * DHHV, update(cfirst[u], rr));
      }
      r += UNROLL * TY;
    }
    for (; r + (UNROLL - 1) * TY < DHQK; r += UNROLL * TY) {
      StatePiece<SBF> c[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) c[u] = load_piece<SBF, NONTEMPORAL>(c_in, cbase + (size_t)(r + u * TY) * DHHV);
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int rr = r + u * TY;
        store_piece<SBF, NONTEMPORAL>(c_out, cbase + (size_t)rr * DHHV, update(c[u], rr));
      }
    }
    for (; r < DHQK; r += TY) {
      const StatePiece<SBF> c = load_piece<SBF, false>(c_in, cbase + (size_t)r * DHHV);
      store_piece<SBF, false>(c_out, cbase + (size_t)r * DHHV, update(c, r));
    }
  }
#pragma unroll
  for (int e = 0; e < VPL; ++e) red[ty * COLS + VPL * tx + e] = acc[e];
  __syncthreads();
  for (int cidx = tid; cidx < COLS; cidx += NTH) {
    if (col0 + cidx < DHHV) {
      float s = 0.f;
#pragma unroll
      for (int y = 0; y < TY; ++y) s += red[y * COLS + cidx];
      s *= inv_den;
      const size_t o = (size_t)bh * DHHV + col0 + cidx;
      store_state_scalar(h, o, dtype_qkv, s);   // fp32, bf16 or fp16
    }
  }
}

template <int COLS, int TY, int UNROLL, bool NONTEMPORAL, int SBF>
static const char* launch_step_t(const void* q, const void* k, const void* v, const void* i, const void* f,
                                 const void* c_in, const void* n_in, const void* m_in, void* h, void* c_out,
                                 void* n_out, void* m_out, int B, int NH, int DHQK, int DHHV, float eps,
                                 int dtype_qkv, int dtype_gates, hipStream_t stream) {
  const size_t smem = (size_t)(2 * DHQK + TY * COLS) * sizeof(float);
  if (smem > 64 * 1024) return "mlstm_hip_step: DHQK too large for the LDS staging";
  dim3 grid((DHHV + COLS - 1) / COLS, B * NH);
  hipLaunchKernelGGL((step_kernel<COLS, TY, UNROLL, NONTEMPORAL, SBF>), grid, dim3((COLS / StatePiece<SBF>::N) * TY), smem,
                     stream, q, k, v, i, f, c_in, n_in, m_in, h, c_out, n_out, m_out, DHQK, DHHV, eps, dtype_qkv,
                     dtype_gates);
  return nullptr;
}

const char* launch_step(const void* q, const void* k, const void* v, const void* i, const void* f,
                        const void* c_in, const void* n_in, const void* m_in, void* h, void* c_out,
                        void* n_out, void* m_out, int B, int NH, int DHQK, int DHHV, float eps,
                        int dtype_qkv, int dtype_gates, int dtype_state, hipStream_t stream) {
  if (B <= 0 || NH <= 0 || DHQK <= 0 || DHHV <= 0) return "mlstm_hip_step: non-positive dimension";
  const bool sbf = dtype_state != 0;
  if (DHHV % (sbf ? 8 : 4) != 0)
    return sbf ? "mlstm_hip_step: DHHV must be a multiple of 8 for a 16-bit state" : "mlstm_hip_step: DHHV must be a multiple of 4";
  if ((long long)B * NH > 65535) return "mlstm_hip_step: B*NH exceeds 65535";
  // Tile shapes from a sweep on MI355X (B = 16/64/256, NH = 8, 256 x 512 fp32 state).  A state larger than the 256 MB
  // memory-side cache streams past the caches with non-temporal accesses: 256-column slices, 8 row groups, 16 rows
  // in flight per lane.  A smaller one is best left cacheable (it is re-read by the next step) and has few
  // workgroups per CU: 128-column slices with 16 row groups, the first 16 rows per lane requested before the
  // prologue.  The crossover was measured between a 268 MB state (cacheable 79 us, streaming 90 us) and a 403 MB
  // state (156 us against 133 us).  A bfloat16 or float16 state uses the same shapes with lanes of eight columns (half as many
  // lanes per row segment), so every lane still moves 16 bytes per access.
  const size_t state_bytes = (size_t)B * NH * DHQK * DHHV * (sbf ? 2 : 4);
  const bool stream_past_cache = state_bytes > ((size_t)320 << 20);
#define MLSTM_STEP_ARGS q, k, v, i, f, c_in, n_in, m_in, h, c_out, n_out, m_out, B, NH, DHQK, DHHV, eps, dtype_qkv, dtype_gates, stream
#define MLSTM_STEP_PICK(COLS_, TY_, UN_, NT_)                                                          \
  {                                                                                                     \
    if (dtype_state == 1) return launch_step_t<COLS_, TY_, UN_, NT_, 1>(MLSTM_STEP_ARGS);               \
    if (dtype_state == 2) return launch_step_t<COLS_, TY_, UN_, NT_, 2>(MLSTM_STEP_ARGS);               \
    return launch_step_t<COLS_, TY_, UN_, NT_, 0>(MLSTM_STEP_ARGS);                                      \
  }
  if (DHHV % 256 == 0 && stream_past_cache) MLSTM_STEP_PICK(256, 8, 16, true)
  if (stream_past_cache) MLSTM_STEP_PICK(128, 8, 8, true)
  MLSTM_STEP_PICK(128, 16, 16, false)
#undef MLSTM_STEP_PICK
#undef MLSTM_STEP_ARGS
}

}  // namespace mlstm
