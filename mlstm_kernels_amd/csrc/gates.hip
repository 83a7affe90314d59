// Gate pre-pass of the chunkwise mLSTM kernels.
//
// Every stabiliser of the chunkwise formulation depends on the gate pre-activations only, never on q/k/v.
// This pass therefore turns (i, f) into the fp32 vectors the matrix kernels consume, so that their inner
// loops are plain scaled GEMM chains with no running-max rescaling:
//
//   per position t of chunk c (chunk length 128, b = inclusive within-chunk cumsum of logsig(f),
//   it = i for the exponential gate, logsig(i) for the sigmoid gate):
//     m_comb[t] = max(b_t + m_{c-1}, b_t + max_{j<=t}(it_j - b_j))          (0 for the sigmoid gate)
//     u[t]      = b_t - m_comb[t]            w[t] = b_t - it_t        => D[t][j] = exp(u[t] - w[j]), j <= t
//     bbar[t]   = exp(b_t + m_{c-1} - m_comb[t])                        (weight of the incoming state)
//     abar[t]   = exp(sum_{u>t} logsig(f_u) + it_t - m_c)               (weight of k_t v_t^T in C_c)
//   per chunk c:  gbar[c] = exp(g_c + m_{c-1} - m_c),  m_c = max(g_c + m_{c-1}, max_t a_t)   (m = 0 for sig)
//
// (formulas of mlstm_kernels/torch/chunkwise/native/fw.py:81-121,171-190 in the reference.)  Positions past
// the sequence end inside the last chunk get logsig(f) = 0 and it = -inf, i.e. they neither decay nor feed
// the state, so any sequence length is handled.
//
// Two launches, each with one workgroup per (batch, head, group of 16 chunks) so that a small batch still fills
// the chip: the first does the within-chunk scans (one wave per chunk); the second scans the (max,+) recurrence of m
// over ALL chunks of its head with one wave (the recurrence is associative and only NC scalars long, so every
// workgroup of a head repeats it rather than waiting for a neighbour) and finishes its own chunks elementwise.
#include "common.h"
#include "kernels.h"

namespace mlstm {

constexpr int kGateThreads = 1024;

template <typename Op>
__device__ __forceinline__ float wave_incl_scan(float x, Op op, float identity) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const float y = __shfl_up(x, o);
    x = lane >= o ? op(y, x) : x;
  }
  (void)identity;
  return x;
}
template <typename Op>
__device__ __forceinline__ float wave_rev_incl_scan(float x, Op op) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const float y = __shfl_down(x, o);
    x = lane + o < 64 ? op(y, x) : x;
  }
  return x;
}

constexpr int kGateChunks = kGateThreads / kWave;  // chunks per workgroup: one wave each

__global__ __launch_bounds__(kGateThreads) void gates_scan_kernel(
    const void* __restrict__ ig, const void* __restrict__ fg, GateBufs gb, int S, int NC, int dtype_gates,
    int sig_gate) {
  const int bh = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = blockIdx.x * kGateChunks + wave;
  if (c >= NC) return;
  const size_t Sp = (size_t)NC * kChunk;
  float* u = gb.u + bh * Sp;          // here: b
  float* wv = gb.w + bh * Sp;
  float* abar = gb.abar + bh * Sp;    // here: a
  float* mcomb = gb.mcomb + bh * Sp;  // here: b + cummax(it - b)
  const float NEG_INF = -__builtin_inff();
  auto add = [](float a, float b) { return a + b; };
  auto mx = [](float a, float b) { return fmaxf(a, b); };

  // within-chunk scans, one wave per chunk, two positions per lane
  const int t0 = c * kChunk + 2 * lane;
  float lf[2], it[2];
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    const int t = t0 + e;
    if (t < S) {
      const size_t o = (size_t)bh * S + t;
      lf[e] = log_sigmoid(load_scalar(fg, o, dtype_gates));
      const float iv = load_scalar(ig, o, dtype_gates);
      it[e] = sig_gate ? log_sigmoid(iv) : iv;
    } else {
      lf[e] = 0.f;
      it[e] = NEG_INF;
    }
  }
  const float pair = lf[0] + lf[1];
  const float incl = wave_incl_scan(pair, add, 0.f);
  const float b1 = incl, b0 = (incl - pair) + lf[0];
  const float g = __shfl(incl, 63);
  const float rincl = wave_rev_incl_scan(pair, add);
  const float suf1 = rincl - pair, suf0 = suf1 + lf[1];
  const float a0 = suf0 + it[0], a1 = suf1 + it[1];
  const float x0 = it[0] - b0, x1 = it[1] - b1;
  const float pm = wave_incl_scan(fmaxf(x0, x1), mx, NEG_INF);
  float pm_excl = __shfl_up(pm, 1);
  if (lane == 0) pm_excl = NEG_INF;
  const float cm0 = fmaxf(pm_excl, x0), cm1 = pm;
  const float am = wave_max(fmaxf(a0, a1));
  *(float2*)(u + t0) = make_float2(b0, b1);
  *(float2*)(mcomb + t0) = make_float2(b0 + cm0, b1 + cm1);
  *(float2*)(abar + t0) = make_float2(a0, a1);
  *(float2*)(wv + t0) = make_float2(b0 - it[0], b1 - it[1]);
  if (lane == 0) {
    gb.graw[(size_t)bh * NC + c] = g;
    gb.amax[(size_t)bh * NC + c] = am;
  }
}

__global__ __launch_bounds__(kGateThreads) void gates_finish_kernel(const float* __restrict__ m0, GateBufs gb,
                                                                    float* __restrict__ m_last, int NC, int sig_gate) {
  __shared__ float msh[kGateChunks + 1];  // m before the chunks of this workgroup, and after its last one
  const int bh = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c_first = blockIdx.x * kGateChunks;
  const int c_end = min(c_first + kGateChunks, NC);
  const size_t Sp = (size_t)NC * kChunk;
  float* u = gb.u + bh * Sp;
  float* abar = gb.abar + bh * Sp;
  float* bbar = gb.bbar + bh * Sp;
  float* mcomb = gb.mcomb + bh * Sp;
  const float* graw = gb.graw + (size_t)bh * NC;
  const float* amax = gb.amax + (size_t)bh * NC;
  float* gbar = gb.gbar + (size_t)bh * NC;
  float* mst = gb.mstates + (size_t)bh * (NC + 1);
  const float NEG_INF = -__builtin_inff();

  // m_c = max(g_c + m_{c-1}, amax_c) over the chunks of the head; (G, A) pairs compose associatively:
  //      (G1, A1) then (G2, A2)  ==  (G1 + G2, max(A1 + G2, A2))
  if (wave == 0) {
    if (sig_gate) {
      for (int c = c_first + lane; c < c_end; c += kWave) {
        mst[c] = 0.f;
        gbar[c] = expf(graw[c]);
      }
      if (lane < kGateChunks + 1) msh[lane] = 0.f;
      if (c_end == NC && lane == 0) {
        mst[NC] = 0.f;
        if (m_last != nullptr) m_last[bh] = 0.f;
      }
    } else {
      const float m_init = m0 != nullptr ? m0[bh] : 0.f;
      const int R = (NC + 63) / 64;
      const int c_lo = min(lane * R, NC), c_hi = min(c_lo + R, NC);
      float G = 0.f, A = NEG_INF;
      for (int c = c_lo; c < c_hi; ++c) {
        const float gc = graw[c];
        A = fmaxf(A + gc, amax[c]);
        G += gc;
      }
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const float Gp = __shfl_up(G, o), Ap = __shfl_up(A, o);
        if (lane >= o) {
          A = fmaxf(Ap + G, A);
          G = Gp + G;
        }
      }
      float Gex = __shfl_up(G, 1), Aex = __shfl_up(A, 1);
      if (lane == 0) {
        Gex = 0.f;
        Aex = NEG_INF;
      }
      float m = fmaxf(m_init + Gex, Aex);
      for (int c = c_lo; c < c_hi; ++c) {
        const float gc = graw[c];
        const float mn = fmaxf(m + gc, amax[c]);
        if (c >= c_first && c < c_end) {  // this workgroup's chunks: publish
          mst[c] = m;
          gbar[c] = expf(gc + m - mn);
          msh[c - c_first] = m;
          msh[c - c_first + 1] = mn;
          if (c == NC - 1) {
            mst[NC] = mn;
            if (m_last != nullptr) m_last[bh] = mn;
          }
        }
        m = mn;
      }
    }
  }
  __syncthreads();

  // elementwise finalisation of this workgroup's chunks
  const size_t t_lo = (size_t)c_first * kChunk, t_hi = (size_t)c_end * kChunk;
  for (size_t t = t_lo + tid; t < t_hi; t += kGateThreads) {
    const int cl = (int)(t / kChunk) - c_first;
    const float mp = msh[cl], mn = msh[cl + 1];
    const float b = u[t], mi = mcomb[t], a = abar[t];
    const float mc = sig_gate ? 0.f : fmaxf(b + mp, mi);
    u[t] = b - mc;
    bbar[t] = expf(b + mp - mc);
    abar[t] = expf(a - mn);
    mcomb[t] = mc;
  }
}

const char* launch_gates(const void* i, const void* f, const float* m0, const GateBufs& gb, float* m_last,
                         int B, int NH, int S, int dtype_gates, int sig_gate, hipStream_t stream) {
  const int NC = (S + kChunk - 1) / kChunk;
  const dim3 grid((NC + kGateChunks - 1) / kGateChunks, B * NH);
  hipLaunchKernelGGL(gates_scan_kernel, grid, dim3(kGateThreads), 0, stream, i, f, gb, S, NC, dtype_gates, sig_gate);
  hipLaunchKernelGGL(gates_finish_kernel, grid, dim3(kGateThreads), 0, stream, m0, gb, m_last, NC, sig_gate);
  return nullptr;
}

// Gate gradients (mlstm_kernels/torch/chunkwise/native/bw.py:320-326 and
// mlstm_kernels/torch/chunkwise/triton_xl_chunk_siging/chunkwise_gates.py:72-100 in the reference):
//   dF[t] = sigmoid(-f_t) * sum_{u >= t} (q_u.dQ_u - k_u.dK_u)     (suffix sum over the WHOLE sequence)
//   dI[t] = k_t.dK_t   (times sigmoid(-i_t) for the sigmoid input gate)
// One workgroup per (batch, head, segment of 2048 positions), two neighbouring positions per thread (coalesced):
// the workgroup first adds up everything behind its segment (a plain strided sum over at most S positions), then
// scans its own segment backwards across lanes and waves.
constexpr int kGradSeg = 2 * kGateThreads;

__global__ __launch_bounds__(kGateThreads) void gate_grads_kernel(GateGradArgs a) {
  __shared__ float wtot[kGateThreads / kWave];
  const int bh = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int S = a.S;
  const size_t Sp = (size_t)a.NC * kChunk;
  const float* qdq = a.qdq + bh * Sp;
  const float* kdk = a.kdk + bh * Sp;
  const size_t tile_stride = (size_t)gridDim.y * Sp;  // the row dots come in one slot per head-dimension tile
  auto diff = [&](int t) {  // q.dQ - k.dK of position t, tiles summed in a fixed order
    float s = 0.f;
    for (int tl = 0; tl < a.ntiles; ++tl) s += qdq[tl * tile_stride + t] - kdk[tl * tile_stride + t];
    return s;
  };
  auto kdot = [&](int t) {
    float s = 0.f;
    for (int tl = 0; tl < a.ntiles; ++tl) s += kdk[tl * tile_stride + t];
    return s;
  };
  const int seg_lo = blockIdx.x * kGradSeg;
  const int seg_hi = min(seg_lo + kGradSeg, S);
  // everything behind this segment
  float part = 0.f;
  for (int t = seg_hi + tid; t < S; t += kGateThreads) part += diff(t);
  part = wave_sum(part);
  if (lane == 0) wtot[wave] = part;
  __syncthreads();
  float after = 0.f;
#pragma unroll
  for (int w = 0; w < kGateThreads / kWave; ++w) after += wtot[w];
  __syncthreads();
  // this segment, backwards
  const int t0 = seg_lo + 2 * tid;
  float kd[2], d[2];
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    kd[e] = t0 + e < S ? kdot(t0 + e) : 0.f;
    d[e] = t0 + e < S ? diff(t0 + e) : 0.f;
  }
  const float pair = d[0] + d[1];
  auto add = [](float x, float y) { return x + y; };
  const float rincl = wave_rev_incl_scan(pair, add);  // sum over lanes >= lane
  if (lane == 0) wtot[wave] = rincl;
  __syncthreads();
  for (int w = wave + 1; w < kGateThreads / kWave; ++w) after += wtot[w];
  float suf[2];
  suf[1] = after + (rincl - pair) + d[1];
  suf[0] = suf[1] + d[0];
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    if (t0 + e < S) {
      const size_t o = (size_t)bh * S + t0 + e;
      const float fv = load_scalar(a.f, o, a.dtype_gates);
      a.dF[o] = suf[e] * (1.f / (1.f + expf(fv)));  // sigmoid(-f)
      float di = kd[e];
      if (a.sig_gate) di *= 1.f / (1.f + expf(load_scalar(a.i, o, a.dtype_gates)));
      a.dI[o] = di;
    }
  }
}

__global__ void fill_zero_kernel(float* p, size_t n) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0.f;
}

const char* launch_gate_grads(const GateGradArgs& a, int BH, hipStream_t stream) {
  if (a.ntiles < 1) return "gate_grads: the row dots need at least one tile slot";
  hipLaunchKernelGGL(gate_grads_kernel, dim3((a.S + kGradSeg - 1) / kGradSeg, BH), dim3(kGateThreads), 0, stream, a);
  return nullptr;
}

const char* launch_fill_zero(float* p, size_t n, hipStream_t stream) {
  const int blocks = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks > 0 ? blocks : 1), dim3(256), 0, stream, p, n);
  return nullptr;
}

}  // namespace mlstm
