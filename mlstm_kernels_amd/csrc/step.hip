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
// owns (b, head, slice of 128 value columns); 32 lanes x 16 B cover one 512-byte row segment and the 8 row
// groups of the workgroup walk the DHQK rows with all loads of an unrolled batch in flight before the first
// use.  The q^T C' column sums are reduced across the 8 row groups through LDS at the end.
#include "common.h"
#include "kernels.h"

namespace mlstm {

constexpr int kStepCols = 128;                // value columns per workgroup
constexpr int kStepTX = kStepCols / 4;        // 32 lanes per row segment (float4 each)
constexpr int kStepTY = 8;                    // row groups
constexpr int kStepThreads = kStepTX * kStepTY;
constexpr int kStepUnroll = 8;

__global__ __launch_bounds__(kStepThreads) void step_kernel(
    const void* __restrict__ q, const void* __restrict__ k, const void* __restrict__ v,
    const void* __restrict__ ig, const void* __restrict__ fg,
    const float* c_in, const float* n_in, const float* m_in,
    void* __restrict__ h, float* c_out, float* n_out, float* m_out,
    int DHQK, int DHHV, float eps, int dtype_qkv, int dtype_gates) {
  extern __shared__ float smem[];
  float* qs = smem;                 // [DHQK] q / sqrt(d)
  float* ik = smem + DHQK;          // [DHQK] i' * k
  float* red = smem + 2 * DHQK;     // [kStepTY][kStepCols] partial column sums, then [8] scalars
  const int bh = blockIdx.y;
  const int col0 = blockIdx.x * kStepCols;
  const int tid = threadIdx.x;
  const int tx = tid % kStepTX, ty = tid / kStepTX;

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
  for (int d = tid; d < DHQK; d += kStepThreads) {
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
  __shared__ float wsum[kStepThreads / kWave];
  if ((tid & 63) == 0) wsum[tid >> 6] = qn_part;
  __syncthreads();
  float qn = 0.f;
#pragma unroll
  for (int w = 0; w < kStepThreads / kWave; ++w) qn += wsum[w];
  const float inv_den = 1.f / (fmaxf(fabsf(qn), expf(-m_new)) + eps);
  if (blockIdx.x == 0 && tid == 0) m_out[bh] = m_new;

  const int col = col0 + 4 * tx;
  const bool col_ok = col < DHHV;  // DHHV % 4 == 0 is checked on the host
  float4 vv = make_float4(0.f, 0.f, 0.f, 0.f);
  if (col_ok) {
    const size_t o = (size_t)bh * DHHV + col;
    if (dtype_qkv == 0) {
      vv = *(const float4*)((const float*)v + o);
    } else {
      const uint2 raw = *(const uint2*)((const uint16_t*)v + o);
      vv.x = __uint_as_float(raw.x << 16);
      vv.y = __uint_as_float(raw.x & 0xffff0000u);
      vv.z = __uint_as_float(raw.y << 16);
      vv.w = __uint_as_float(raw.y & 0xffff0000u);
    }
  }
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  if (col_ok) {
    const f32x4 v4 = {vv.x, vv.y, vv.z, vv.w};
    const float* cin = c_in + (size_t)bh * DHQK * DHHV + col;
    float* cout = c_out + (size_t)bh * DHQK * DHHV + col;
    int r = ty;
    for (; r + (kStepUnroll - 1) * kStepTY < DHQK; r += kStepUnroll * kStepTY) {
      f32x4 c[kStepUnroll];
#pragma unroll
      for (int u = 0; u < kStepUnroll; ++u)
        c[u] = __builtin_nontemporal_load((const f32x4*)(cin + (size_t)(r + u * kStepTY) * DHHV));
#pragma unroll
      for (int u = 0; u < kStepUnroll; ++u) {
        const int rr = r + u * kStepTY;
        const f32x4 o = fa * c[u] + ik[rr] * v4;
        __builtin_nontemporal_store(o, (f32x4*)(cout + (size_t)rr * DHHV));
        acc += qs[rr] * o;
      }
    }
    for (; r < DHQK; r += kStepTY) {
      const f32x4 c = *(const f32x4*)(cin + (size_t)r * DHHV);
      const f32x4 o = fa * c + ik[r] * v4;
      *(f32x4*)(cout + (size_t)r * DHHV) = o;
      acc += qs[r] * o;
    }
  }
  *(f32x4*)(red + ty * kStepCols + 4 * tx) = acc;
  __syncthreads();
  if (tid < kStepCols && col0 + tid < DHHV) {
    float s = 0.f;
#pragma unroll
    for (int y = 0; y < kStepTY; ++y) s += red[y * kStepCols + tid];
    s *= inv_den;
    const size_t o = (size_t)bh * DHHV + col0 + tid;
    if (dtype_qkv == 0) ((float*)h)[o] = s;
    else ((uint16_t*)h)[o] = f32_to_bf16_bits(s);
  }
}

const char* launch_step(const void* q, const void* k, const void* v, const void* i, const void* f,
                        const float* c_in, const float* n_in, const float* m_in, void* h, float* c_out,
                        float* n_out, float* m_out, int B, int NH, int DHQK, int DHHV, float eps,
                        int dtype_qkv, int dtype_gates, hipStream_t stream) {
  if (B <= 0 || NH <= 0 || DHQK <= 0 || DHHV <= 0) return "mlstm_hip_step: non-positive dimension";
  if (DHHV % 4 != 0) return "mlstm_hip_step: DHHV must be a multiple of 4";
  if ((long long)B * NH > 65535) return "mlstm_hip_step: B*NH exceeds 65535";
  const size_t smem = (size_t)(2 * DHQK + kStepTY * kStepCols) * sizeof(float);
  if (smem > 64 * 1024) return "mlstm_hip_step: DHQK too large for the LDS staging (max 7168)";
  dim3 grid((DHHV + kStepCols - 1) / kStepCols, B * NH);
  hipLaunchKernelGGL(step_kernel, grid, dim3(kStepThreads), smem, stream, q, k, v, i, f, c_in, n_in, m_in, h,
                     c_out, n_out, m_out, DHQK, DHHV, eps, dtype_qkv, dtype_gates);
  return nullptr;
}

}  // namespace mlstm
