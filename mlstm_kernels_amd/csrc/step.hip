// Fused recurrent decode step of the mLSTM (exponential input gate), one token per (batch, head).
//
//   m' = max(logsig(f) + m, i)          f' = exp(logsig(f) + m - m')      i' = exp(i - m')
//   C' = f' C + i' k v^T                n' = f' n + i' k
//   h  = (q/sqrt(d))^T C' / (max(|q/sqrt(d) . n'|, exp(-m')) + eps)
//
// (math of mlstm_kernels/torch/recurrent/native_step.py:69-95 in the reference; everything in fp32.)
//
// The step is a pure stream over the fp32 state C (DHQK x DHHV per head): one read and one write of every
// element, 0.75 flop per byte, so it is laid out for HBM bandwidth only -- no matrix cores.  A workgroup
// owns (b, head, slice of COLS value columns); COLS/4 lanes x 16 B cover one contiguous row segment and the TY
// row groups of the workgroup walk the DHQK rows with all loads of an unrolled batch in flight before the first
// use.  The q^T C' column sums are reduced across the row groups through LDS at the end.
#include "common.h"
#include "kernels.h"

namespace mlstm {

template <int COLS, int TY, int UNROLL, bool NONTEMPORAL>
__global__ __launch_bounds__((COLS / 4) * TY) void step_kernel(
    const void* __restrict__ q, const void* __restrict__ k, const void* __restrict__ v,
    const void* __restrict__ ig, const void* __restrict__ fg,
    const float* c_in, const float* n_in, const float* m_in,
    void* __restrict__ h, float* c_out, float* n_out, float* m_out,
    int DHQK, int DHHV, float eps, int dtype_qkv, int dtype_gates) {
  constexpr int TX = COLS / 4;
  constexpr int NTH = TX * TY;
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
  const int col = col0 + 4 * tx;
  const bool col_ok = col < DHHV;  // DHHV % 4 == 0 is checked on the host
  const float* cin = c_in + (size_t)bh * DHQK * DHHV + col;
  float* cout = c_out + (size_t)bh * DHQK * DHHV + col;
  const bool have_first = !NONTEMPORAL && col_ok && ty + (UNROLL - 1) * TY < DHQK;
  f32x4 cfirst[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const f32x4 z = {0.f, 0.f, 0.f, 0.f};
    const f32x4* p = (const f32x4*)(cin + (size_t)(ty + u * TY) * DHHV);
    cfirst[u] = have_first ? *p : z;
  }

  const float fpre = load_scalar(fg, bh, dtype_gates);
  const float ipre = load_scalar(ig, bh, dtype_gates);
  const float m_old = m_in[bh];
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
    const float nd = fa * n_in[o] + ia * kd;
    qs[d] = qd;
    ik[d] = ia * kd;
    qn_part += qd * nd;
    if (blockIdx.x == 0) n_out[o] = nd;
  }
  qn_part = wave_sum(qn_part);
  __shared__ float wsum[(NTH + kWave - 1) / kWave];
  if ((tid & 63) == 0) wsum[tid >> 6] = qn_part;
  __syncthreads();
  float qn = 0.f;
#pragma unroll
  for (int w = 0; w < (NTH + kWave - 1) / kWave; ++w) qn += wsum[w];
  const float inv_den = 1.f / (fmaxf(fabsf(qn), expf(-m_new)) + eps);
  if (blockIdx.x == 0 && tid == 0) m_out[bh] = m_new;

  f32x4 v4 = {0.f, 0.f, 0.f, 0.f};
  if (col_ok) {
    const size_t o = (size_t)bh * DHHV + col;
    if (dtype_qkv == 0) {
      v4 = *(const f32x4*)((const float*)v + o);
    } else {
      const uint2 raw = *(const uint2*)((const uint16_t*)v + o);
      v4[0] = __uint_as_float(raw.x << 16);
      v4[1] = __uint_as_float(raw.x & 0xffff0000u);
      v4[2] = __uint_as_float(raw.y << 16);
      v4[3] = __uint_as_float(raw.y & 0xffff0000u);
    }
  }
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  if (col_ok) {
    int r = ty;
    if (have_first) {
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int rr = r + u * TY;
        const f32x4 o = fa * cfirst[u] + ik[rr] * v4;
        *(f32x4*)(cout + (size_t)rr * DHHV) = o;
        acc += qs[rr] * o;
      }
      r += UNROLL * TY;
    }
    for (; r + (UNROLL - 1) * TY < DHQK; r += UNROLL * TY) {
      f32x4 c[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const f32x4* p = (const f32x4*)(cin + (size_t)(r + u * TY) * DHHV);
        c[u] = NONTEMPORAL ? __builtin_nontemporal_load(p) : *p;
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int rr = r + u * TY;
        const f32x4 o = fa * c[u] + ik[rr] * v4;
        f32x4* p = (f32x4*)(cout + (size_t)rr * DHHV);
        if (NONTEMPORAL) __builtin_nontemporal_store(o, p);
        else *p = o;
        acc += qs[rr] * o;
      }
    }
    for (; r < DHQK; r += TY) {
      const f32x4 c = *(const f32x4*)(cin + (size_t)r * DHHV);
      const f32x4 o = fa * c + ik[r] * v4;
      *(f32x4*)(cout + (size_t)r * DHHV) = o;
      acc += qs[r] * o;
    }
  }
  *(f32x4*)(red + ty * COLS + 4 * tx) = acc;
  __syncthreads();
  for (int cidx = tid; cidx < COLS; cidx += NTH) {
    if (col0 + cidx < DHHV) {
      float s = 0.f;
#pragma unroll
      for (int y = 0; y < TY; ++y) s += red[y * COLS + cidx];
      s *= inv_den;
      const size_t o = (size_t)bh * DHHV + col0 + cidx;
      if (dtype_qkv == 0) ((float*)h)[o] = s;
      else ((uint16_t*)h)[o] = f32_to_bf16_bits(s);
    }
  }
}

template <int COLS, int TY, int UNROLL, bool NONTEMPORAL>
static const char* launch_step_t(const void* q, const void* k, const void* v, const void* i, const void* f,
                                 const float* c_in, const float* n_in, const float* m_in, void* h, float* c_out,
                                 float* n_out, float* m_out, int B, int NH, int DHQK, int DHHV, float eps,
                                 int dtype_qkv, int dtype_gates, hipStream_t stream) {
  const size_t smem = (size_t)(2 * DHQK + TY * COLS) * sizeof(float);
  if (smem > 64 * 1024) return "mlstm_hip_step: DHQK too large for the LDS staging";
  dim3 grid((DHHV + COLS - 1) / COLS, B * NH);
  hipLaunchKernelGGL((step_kernel<COLS, TY, UNROLL, NONTEMPORAL>), grid, dim3((COLS / 4) * TY), smem, stream, q, k, v,
                     i, f, c_in, n_in, m_in, h, c_out, n_out, m_out, DHQK, DHHV, eps, dtype_qkv, dtype_gates);
  return nullptr;
}

#ifndef MLSTM_STEP_NO_DEFAULT_LAUNCHER
const char* launch_step(const void* q, const void* k, const void* v, const void* i, const void* f,
                        const float* c_in, const float* n_in, const float* m_in, void* h, float* c_out,
                        float* n_out, float* m_out, int B, int NH, int DHQK, int DHHV, float eps,
                        int dtype_qkv, int dtype_gates, hipStream_t stream) {
  if (B <= 0 || NH <= 0 || DHQK <= 0 || DHHV <= 0) return "mlstm_hip_step: non-positive dimension";
  if (DHHV % 4 != 0) return "mlstm_hip_step: DHHV must be a multiple of 4";
  if ((long long)B * NH > 65535) return "mlstm_hip_step: B*NH exceeds 65535";
  // Tile shapes from a sweep on MI355X (B = 16/64/256, NH = 8, 256 x 512 state).  A state larger than the 256 MB
  // memory-side cache streams past the caches with non-temporal accesses: 256-column slices, 8 row groups, 16 rows
  // in flight per lane.  A smaller one is best left cacheable (it is re-read by the next step) and has few
  // workgroups per CU: 128-column slices with 16 row groups, the first 16 rows per lane requested before the
  // prologue.  The crossover was measured between a 268 MB state (cacheable 79 us, streaming 90 us) and a 403 MB
  // state (156 us against 133 us).
  const size_t state_bytes = (size_t)B * NH * DHQK * DHHV * sizeof(float);
  const bool stream_past_cache = state_bytes > ((size_t)320 << 20);
#define MLSTM_STEP_ARGS q, k, v, i, f, c_in, n_in, m_in, h, c_out, n_out, m_out, B, NH, DHQK, DHHV, eps, dtype_qkv, dtype_gates, stream
  if (DHHV % 256 == 0) {
    if (stream_past_cache) return launch_step_t<256, 8, 16, true>(MLSTM_STEP_ARGS);
    return launch_step_t<128, 16, 16, false>(MLSTM_STEP_ARGS);
  }
  if (stream_past_cache) return launch_step_t<128, 8, 8, true>(MLSTM_STEP_ARGS);
  return launch_step_t<128, 16, 16, false>(MLSTM_STEP_ARGS);
#undef MLSTM_STEP_ARGS
}
#endif

}  // namespace mlstm
