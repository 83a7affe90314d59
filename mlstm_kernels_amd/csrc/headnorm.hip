// Backward of the head norm that the forward kernel fuses into the H epilogue (the reference states the norm in
// mlstm_kernels/utils/analysis/transfer_behavior/_norm_layers.py:11-35: layer_normalize / rms_normalize over the last
// dimension, fp32 reductions, no scale parameters).
//
//   layer:  y = (x - mean) * rstd     dx = rstd * (dy - mean_D(dy) - y * mean_D(dy * y))
//   rms  :  y = x * rstd              dx = rstd * (dy - y * mean_D(dy * y))
//
// Needs only the normalised rows y (what the forward wrote), the per-row rstd and the incoming gradient: the
// un-normalised H is never materialised.  One wave per row, rows of D <= 512 bf16 or fp16 values (D / 64 per lane, fetched as
// one 16-byte vector when D = 512); a pure streaming kernel (reads 2 rows, writes 1).
#include "common.h"
#include "kernels.h"

namespace mlstm {

template <int VPL, bool F16>  // values per lane: D = 64 * VPL; rows of float16 (F16) or bfloat16 values
__global__ __launch_bounds__(256) void head_norm_bw_kernel(HeadNormBwArgs a) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const size_t row = (size_t)blockIdx.x * 4 + wave;
  if (row >= a.rows) return;
  const uint16_t* dy_p = a.dY + row * a.D + lane * VPL;
  const uint16_t* y_p = a.Y + row * a.D + lane * VPL;
  float dy[VPL], y[VPL];
  if constexpr (VPL == 8) {
    const uint4 d4 = *(const uint4*)dy_p, y4 = *(const uint4*)y_p;
    const uint32_t dw[4] = {d4.x, d4.y, d4.z, d4.w}, yw[4] = {y4.x, y4.y, y4.z, y4.w};
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      dy[2 * p] = lo2<F16>(dw[p]);
      dy[2 * p + 1] = hi2<F16>(dw[p]);
      y[2 * p] = lo2<F16>(yw[p]);
      y[2 * p + 1] = hi2<F16>(yw[p]);
    }
  } else {
#pragma unroll
    for (int e = 0; e < VPL; ++e) {
      dy[e] = elem_to_f32<F16>(dy_p[e]);
      y[e] = elem_to_f32<F16>(y_p[e]);
    }
  }
  float s1 = 0.f, s2 = 0.f;
#pragma unroll
  for (int e = 0; e < VPL; ++e) {
    s1 += dy[e];
    s2 += dy[e] * y[e];
  }
  s1 = wave_sum(s1) / (float)a.D;
  s2 = wave_sum(s2) / (float)a.D;
  if (a.kind == 2) s1 = 0.f;
  const float rs = a.rstd[row];
  uint16_t* dx_p = a.dX + row * a.D + lane * VPL;
  if constexpr (VPL == 8) {
    uint32_t o[4];
#pragma unroll
    for (int p = 0; p < 4; ++p)
      o[p] = pack2<F16>(rs * (dy[2 * p] - s1 - y[2 * p] * s2), rs * (dy[2 * p + 1] - s1 - y[2 * p + 1] * s2));
    *(uint4*)dx_p = make_uint4(o[0], o[1], o[2], o[3]);
  } else {
#pragma unroll
    for (int e = 0; e < VPL; ++e) dx_p[e] = f32_to_elem<F16>(rs * (dy[e] - s1 - y[e] * s2));
  }
}

const char* launch_head_norm_bw(const HeadNormBwArgs& a, hipStream_t stream) {
  if (a.kind != 1 && a.kind != 2) return "head_norm_bw: unknown norm code";
  if (a.rows == 0) return nullptr;
  if (a.rows > (size_t)4 * 2147483647) return "head_norm_bw: too many rows";
  const dim3 grid((unsigned)((a.rows + 3) / 4)), block(256);
#define MLSTM_HEAD_NORM_BW(VPL_)                                                                          \
  if (a.f16) hipLaunchKernelGGL((head_norm_bw_kernel<VPL_, true>), grid, block, 0, stream, a);              \
  else hipLaunchKernelGGL((head_norm_bw_kernel<VPL_, false>), grid, block, 0, stream, a)
  switch (a.D) {
    case 64: MLSTM_HEAD_NORM_BW(1); break;
    case 128: MLSTM_HEAD_NORM_BW(2); break;
    case 256: MLSTM_HEAD_NORM_BW(4); break;
    case 512: MLSTM_HEAD_NORM_BW(8); break;
    default: return "head_norm_bw: D must be 64, 128, 256 or 512";
  }
#undef MLSTM_HEAD_NORM_BW
  return nullptr;
}

}  // namespace mlstm
