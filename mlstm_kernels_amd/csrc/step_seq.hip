// Recurrent mLSTM over T tokens in ONE launch: the step of step.hip repeated with the state held on chip.
//
//   for t = 0 .. T-1:   m' = max(logsig(f_t) + m, i_t)      f' = exp(logsig(f_t) + m - m')     i' = exp(i_t - m')
//                       C  = f' C + i' k_t v_t^T             n  = f' n + i' k_t
//                       h_t = (q_t/sqrt(d))^T C / (max(|q_t/sqrt(d) . n|, exp(-m')) + eps)
//
// (the token loop of mlstm_kernels/torch/recurrent/native_sequence.py:13-122 around the step of
// native_step.py:69-95 in the reference; everything in fp32.)
//
// A token loop of single-step launches moves the whole fp32 state through HBM once each way per token.  Here a
// workgroup -- ONE wave -- owns (batch, head, 8*CPT value columns) for the whole sequence: its DHQK x 8*CPT slice of C
// lives in registers (up to 128 per lane), n and m are carried by every workgroup of the head on its own (they are
// tiny), and the state is read once before the first token and written once after the last.  With the state on chip
// the loop is bound by instruction issue and by the latency of one token's dependent steps, so the kernel is laid out
// to keep both short and to keep as much state per CU in registers as the register file allows (three waves per SIMD
// at DHQK = 256: three quarters of the file hold state):
//   * lane (column group c, row group g) holds rows g*RPT .. g*RPT + RPT-1 of CPT neighbouring columns; the eight row
//     groups of a column are eight neighbouring lanes, so the column sums q^T C are finished with three cross-lane
//     additions inside the wave (no LDS, no barrier), and the state is loaded and stored in 16-byte pieces of full
//     128-byte lines;
//   * the gate recurrence does not depend on C: for 64 tokens at a time all lanes evaluate logsig(f) in parallel,
//     one lane runs the max recurrence, and all lanes turn it into tables f', i', exp(-m') in LDS -- the token
//     loop reads three table entries instead of evaluating a logarithm and three exponentials per lane and token;
//   * q_t, k_t and this lane's v_t are requested PF tokens ahead; q/sqrt(d) and i'k are staged in LDS (alternating
//     buffers), q.n' is reduced across the wave with cross-lane additions.
#include "common.h"
#include "kernels.h"

namespace mlstm {

namespace {
// x + (x of the lane selected by the DPP control word), all lanes active
template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
  const int y = __builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, false);
  return x + __int_as_float(y);
}
constexpr int kDppXor1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane i <-> 7 - i inside each group of 8
constexpr int kDppMirror = 0x140;      // lane i <-> 15 - i inside each row of 16
}  // namespace

// waves per SIMD the register budget is cut for: the state slice takes RPT * CPT registers per lane
#define STEP_SEQ_WPE(REGS_) ((REGS_) <= 64 ? 3 : 2)
template <int RPT, int CPT, bool VEC, int QDT>
__global__ __launch_bounds__(64)
    __attribute__((amdgpu_waves_per_eu(STEP_SEQ_WPE(RPT * CPT), STEP_SEQ_WPE(RPT * CPT)))) void step_seq_kernel(
    const void* __restrict__ q, const void* __restrict__ k, const void* __restrict__ v,
    const void* __restrict__ ig, const void* __restrict__ fg,
    const void* c_in, const void* n_in, const void* m_in,
    void* __restrict__ h, void* c_out, void* n_out, void* m_out,
    int T, int DHQK, int DHHV, float eps, int dtype_gates, int dtype_state) {
  constexpr int NG = 8;                       // row groups per column (neighbouring lanes)
  constexpr int COLS = 8 * CPT;               // value columns per workgroup
  constexpr int DMAX = RPT * NG;              // largest DHQK this instantiation holds
  constexpr int NDJ = DMAX / kWave;           // q/k/n entries per lane
  constexpr int RS = RPT + 4;                 // LDS stride of a row group (its 16-byte reads fall into distinct banks)
  constexpr int PF = 2;                       // tokens in flight
  constexpr int GB = kWave;                   // tokens per block of the gate tables
  static_assert(DMAX % kWave == 0 && RPT % 4 == 0, "rows are dealt in fours, q/k entries in whole waves");
  __shared__ __align__(16) float qs[2][NG * RS];  // q_t / sqrt(d), row r at (r / RPT) * RS + r % RPT
  __shared__ __align__(16) float ik[2][NG * RS];  // i' * k_t
  __shared__ float tab_f[GB], tab_i[GB], tab_e[GB], tab_m[GB + 1];
  const int bh = blockIdx.y;
  const int col0 = blockIdx.x * COLS;
  const int lane = threadIdx.x;
  const int g = lane % NG, cl = lane / NG;
  const int col = col0 + CPT * cl;            // first of this lane's CPT columns
  const float scale = rsqrtf((float)DHQK);
  // VEC: whole 16-byte pieces (CPT = 4 and DHHV a multiple of 4: every row segment of a lane is aligned and either
  // inside the matrix or outside)
  constexpr bool vec_ok = VEC;
  static_assert(!VEC || CPT == 4, "16-byte pieces are four columns");

  // ---- state slice into registers; rows past DHQK and columns past DHHV stay zero (their q and k entries in LDS
  // resp. their v entries are zero as well)
  // (loads are unconditional from clamped addresses, the result is selected afterwards: no branches around them)
  float C[RPT][CPT];
  const bool col_in = col < DHHV;
  const bool sbf = dtype_state != 0;  // states in and out in bfloat16 or float16 (fp32 in registers between the tokens)
#pragma unroll
  for (int u = 0; u < RPT; ++u) {
    const int r = g * RPT + u;
    const size_t row = ((size_t)bh * DHQK + min(r, DHQK - 1)) * DHHV;
    if constexpr (VEC) {
      float x[4];
      if (sbf) {
        const uint2 raw = *(const uint2*)((const uint16_t*)c_in + row + (col_in ? col : 0));
        unpack_state2(raw.x, dtype_state, x[0], x[1]);
        unpack_state2(raw.y, dtype_state, x[2], x[3]);
      } else {
        const f32x4 raw = *(const f32x4*)((const float*)c_in + row + (col_in ? col : 0));
#pragma unroll
        for (int e = 0; e < 4; ++e) x[e] = raw[e];
      }
#pragma unroll
      for (int e = 0; e < CPT; ++e) C[u][e] = (r < DHQK && col_in) ? x[e & 3] : 0.f;
    } else {
#pragma unroll
      for (int e = 0; e < CPT; ++e) {
        const float x = load_state_scalar(c_in, row + min(col + e, DHHV - 1), dtype_state);
        C[u][e] = (r < DHQK && col + e < DHHV) ? x : 0.f;
      }
    }
  }
  float nreg[NDJ];
#pragma unroll
  for (int j = 0; j < NDJ; ++j) {
    const int d = lane + j * kWave;
    nreg[j] = d < DHQK ? load_state_scalar(n_in, (size_t)bh * DHQK + d, dtype_state) : 0.f;
  }
  for (int x = lane; x < 2 * NG * RS; x += kWave) {
    (&qs[0][0])[x] = 0.f;
    (&ik[0][0])[x] = 0.f;
  }
  float m = load_state_scalar(m_in, bh, dtype_state);

  // ---- token inputs, PF tokens ahead, in a ring that is shifted by one slot per token.  Tokens past the end
  // re-request the last one (nobody uses them): an unconditional load keeps the ring in registers.
  // Addresses are a uniform base (scalar registers, advanced per token by the scalar unit) plus a constant 32-bit
  // byte offset per lane.
  float qv[PF][NDJ], kv[PF][NDJ], vv[PF][CPT];
  constexpr bool BF16 = QDT != 0;      // q/k/v and h are 16-bit values: bfloat16 (QDT 1) or float16 (QDT 2)
  constexpr bool QF16 = QDT == 2;
  constexpr uint32_t ESZ = BF16 ? 2 : 4;
  uint32_t qoff[NDJ], voff[CPT];
#pragma unroll
  for (int j = 0; j < NDJ; ++j) qoff[j] = (uint32_t)min(lane + j * kWave, DHQK - 1) * ESZ;
#pragma unroll
  for (int e = 0; e < CPT; ++e) voff[e] = (uint32_t)min(col + e, DHHV - 1) * ESZ;
  const char* const q_bh = (const char*)q + (size_t)bh * T * DHQK * ESZ;
  const char* const k_bh = (const char*)k + (size_t)bh * T * DHQK * ESZ;
  const char* const v_bh = (const char*)v + (size_t)bh * T * DHHV * ESZ;
  auto ld = [&](const char* base, uint32_t off) -> float {
    if constexpr (BF16) return elem_to_f32<QF16>(*(const uint16_t*)(base + off));
    else return *(const float*)(base + off);
  };
  auto fetch = [&](int t_, float (&qd)[NDJ], float (&kd)[NDJ], float (&vc)[CPT]) {
    const int t = min(t_, T - 1);
    const char* const qt = q_bh + (size_t)t * DHQK * ESZ;
    const char* const kt = k_bh + (size_t)t * DHQK * ESZ;
    const char* const vt = v_bh + (size_t)t * DHHV * ESZ;
#pragma unroll
    for (int j = 0; j < NDJ; ++j) {
      qd[j] = ld(qt, qoff[j]);
      kd[j] = ld(kt, qoff[j]);
    }
    if constexpr (VEC) {
      // four neighbouring columns in one piece (past the last column: the piece at column 0, zeroed below)
      if constexpr (BF16) {
        const uint2 raw = *(const uint2*)(vt + (col_in ? voff[0] : 0u));
        vc[0] = lo2<QF16>(raw.x);
        vc[1 % CPT] = hi2<QF16>(raw.x);
        vc[2 % CPT] = lo2<QF16>(raw.y);
        vc[3 % CPT] = hi2<QF16>(raw.y);
      } else {
        const f32x4 raw = *(const f32x4*)(vt + (col_in ? voff[0] : 0u));
#pragma unroll
        for (int e = 0; e < CPT; ++e) vc[e] = raw[e & 3];
      }
#pragma unroll
      for (int e = 0; e < CPT; ++e) vc[e] = col_in ? vc[e] : 0.f;
    } else {
#pragma unroll
      for (int e = 0; e < CPT; ++e) {
        const float x = ld(vt, voff[e]);
        vc[e] = col + e < DHHV ? x : 0.f;
      }
    }
  };
#pragma unroll
  for (int p = 0; p < PF; ++p) fetch(p, qv[p], kv[p], vv[p]);

  for (int t0 = 0; t0 < T; t0 += GB) {
    const int nb = min(GB, T - t0);
    // ---- gate tables of tokens t0 .. t0 + nb - 1
    __syncthreads();  // the previous block's tables are no longer read
    float lf = 0.f, ii = 0.f;
    if (lane < nb) {
      const size_t o = (size_t)bh * T + t0 + lane;
      lf = log_sigmoid(load_scalar(fg, o, dtype_gates));
      ii = load_scalar(ig, o, dtype_gates);
      tab_f[lane] = lf;
      tab_i[lane] = ii;
    }
    __syncthreads();
    if (lane == 0) {
      float mm = m;
      tab_m[0] = mm;
      for (int j = 0; j < nb; ++j) {
        mm = fmaxf(tab_f[j] + mm, tab_i[j]);
        tab_m[j + 1] = mm;
      }
    }
    __syncthreads();
    if (lane < nb) {
      const float m_prev = tab_m[lane], m_new = tab_m[lane + 1];
      tab_f[lane] = expf(lf + m_prev - m_new);
      tab_i[lane] = expf(ii - m_new);
      tab_e[lane] = expf(-m_new);
    }
    m = tab_m[nb];
    __syncthreads();
    // ---- the tokens of the block
#pragma unroll 1
    for (int tb = 0; tb < nb; ++tb) {
      const int t = t0 + tb;
      const int buf = t & 1;
      const float fa = tab_f[tb], ia = tab_i[tb], em = tab_e[tb];
      float qn = 0.f;
#pragma unroll
      for (int j = 0; j < NDJ; ++j) {
        const int d = lane + j * kWave;
        if (d < DHQK) {
          const float qsc = qv[0][j] * scale;
          const float nd = fa * nreg[j] + ia * kv[0][j];
          nreg[j] = nd;
          const int o = (d / RPT) * RS + d % RPT;
          qs[buf][o] = qsc;
          ik[buf][o] = ia * kv[0][j];
          qn += qsc * nd;
        }
      }
      float vcur[CPT];
#pragma unroll
      for (int e = 0; e < CPT; ++e) vcur[e] = vv[0][e];
      // shift the ring and request token t + PF into its last slot
#pragma unroll
      for (int p = 0; p + 1 < PF; ++p) {
#pragma unroll
        for (int j = 0; j < NDJ; ++j) {
          qv[p][j] = qv[p + 1][j];
          kv[p][j] = kv[p + 1][j];
        }
#pragma unroll
        for (int e = 0; e < CPT; ++e) vv[p][e] = vv[p + 1][e];
      }
      fetch(t + PF, qv[PF - 1], kv[PF - 1], vv[PF - 1]);
      // q.n' over the whole head: rows of 16 lanes by cross-lane additions, the four rows through the scalar unit
      qn = dpp_add<kDppXor1>(qn);
      qn = dpp_add<kDppXor2>(qn);
      qn = dpp_add<kDppHalfMirror>(qn);
      qn = dpp_add<kDppMirror>(qn);
      {
        const int b = __float_as_int(qn);
        qn = (__int_as_float(__builtin_amdgcn_readlane(b, 0)) + __int_as_float(__builtin_amdgcn_readlane(b, 16))) +
             (__int_as_float(__builtin_amdgcn_readlane(b, 32)) + __int_as_float(__builtin_amdgcn_readlane(b, 48)));
      }
      const float inv_den = 1.f / (fmaxf(fabsf(qn), em) + eps);
      __syncthreads();  // one wave: orders the LDS writes above before the reads below
      float acc[CPT];
#pragma unroll
      for (int e = 0; e < CPT; ++e) acc[e] = 0.f;
      const float* qrow = &qs[buf][g * RS];
      const float* krow = &ik[buf][g * RS];
      // the staged rows are read one group of four ahead of their use; the scheduling barrier keeps the compiler from
      // hoisting all reads of a token to the front (which would need more registers than the state leaves)
      float4 q4 = *(const float4*)qrow, k4 = *(const float4*)krow;
#pragma unroll
      for (int u4 = 0; u4 < RPT / 4; ++u4) {
        const float qq[4] = {q4.x, q4.y, q4.z, q4.w};
        const float kk[4] = {k4.x, k4.y, k4.z, k4.w};
        if (u4 + 1 < RPT / 4) {
          q4 = *(const float4*)(qrow + 4 * (u4 + 1));
          k4 = *(const float4*)(krow + 4 * (u4 + 1));
        }
#pragma unroll
        for (int x = 0; x < 4; ++x)
#pragma unroll
          for (int e = 0; e < CPT; ++e) {
            // decay in place, then accumulate in place (two-address instructions: the state never changes registers)
            C[4 * u4 + x][e] *= fa;
            C[4 * u4 + x][e] = __builtin_fmaf(kk[x], vcur[e], C[4 * u4 + x][e]);
            acc[e] = __builtin_fmaf(qq[x], C[4 * u4 + x][e], acc[e]);
          }
        __builtin_amdgcn_sched_barrier(0);
      }
      // column sums over the eight row groups (eight neighbouring lanes)
#pragma unroll
      for (int e = 0; e < CPT; ++e) {
        acc[e] = dpp_add<kDppXor1>(acc[e]);
        acc[e] = dpp_add<kDppXor2>(acc[e]);
        acc[e] = dpp_add<kDppHalfMirror>(acc[e]);
      }
      if (g == 0) {
        const size_t o = ((size_t)bh * T + t) * DHHV + col;
        if constexpr (vec_ok) {
          if (col_in) {
            if constexpr (!BF16) {
              const f32x4 y = {acc[0] * inv_den, acc[1 % CPT] * inv_den, acc[2 % CPT] * inv_den, acc[3 % CPT] * inv_den};
              *(f32x4*)((float*)h + o) = y;
            } else {
              *(uint2*)((uint16_t*)h + o) = make_uint2(pack2<QF16>(acc[0] * inv_den, acc[1 % CPT] * inv_den),
                                                       pack2<QF16>(acc[2 % CPT] * inv_den, acc[3 % CPT] * inv_den));
            }
          }
        } else {
#pragma unroll
          for (int e = 0; e < CPT; ++e)
            if (col + e < DHHV) {
              const float s = acc[e] * inv_den;
              if constexpr (!BF16) ((float*)h)[o + e] = s;
              else ((uint16_t*)h)[o + e] = f32_to_elem<QF16>(s);
            }
        }
      }
    }
  }

  // ---- state out (C may be updated in place: this workgroup read its whole slice before the first token)
#pragma unroll
  for (int u = 0; u < RPT; ++u) {
    const int r = g * RPT + u;
    if (r < DHQK) {
      const size_t row = ((size_t)bh * DHQK + r) * DHHV;
      if constexpr (vec_ok) {
        if (col_in) {
          if (sbf) {
            *(uint2*)((uint16_t*)c_out + row + col) =
                make_uint2(pack_state2(C[u][0], C[u][1 % CPT], dtype_state), pack_state2(C[u][2 % CPT], C[u][3 % CPT], dtype_state));
          } else {
            const f32x4 y = {C[u][0], C[u][1 % CPT], C[u][2 % CPT], C[u][3 % CPT]};
            *(f32x4*)((float*)c_out + row + col) = y;
          }
        }
      } else {
#pragma unroll
        for (int e = 0; e < CPT; ++e)
          if (col + e < DHHV) store_state_scalar(c_out, row + col + e, dtype_state, C[u][e]);
      }
    }
  }
  if (blockIdx.x == 0) {
#pragma unroll
    for (int j = 0; j < NDJ; ++j) {
      const int d = lane + j * kWave;
      if (d < DHQK) store_state_scalar(n_out, (size_t)bh * DHQK + d, dtype_state, nreg[j]);
    }
    if (lane == 0) store_state_scalar(m_out, bh, dtype_state, m);
  }
}

template <int RPT, int CPT, bool VEC, int QDT>
static const char* launch_step_seq_t(const void* q, const void* k, const void* v, const void* i, const void* f,
                                     const void* c_in, const void* n_in, const void* m_in, void* h, void* c_out,
                                     void* n_out, void* m_out, int B, int NH, int T, int DHQK, int DHHV, float eps,
                                     int dtype_qkv, int dtype_gates, int dtype_state, hipStream_t stream) {
  constexpr int COLS = 8 * CPT;
  dim3 grid((DHHV + COLS - 1) / COLS, B * NH);
  hipLaunchKernelGGL((step_seq_kernel<RPT, CPT, VEC, QDT>), grid, dim3(64), 0, stream, q, k, v, i, f, c_in, n_in, m_in, h,
                     c_out, n_out, m_out, T, DHQK, DHHV, eps, dtype_gates, dtype_state);
  return nullptr;
}

const char* launch_step_seq(const void* q, const void* k, const void* v, const void* i, const void* f,
                            const void* c_in, const void* n_in, const void* m_in, void* h, void* c_out,
                            void* n_out, void* m_out, int B, int NH, int T, int DHQK, int DHHV, float eps,
                            int dtype_qkv, int dtype_gates, int dtype_state, hipStream_t stream) {
  if (B <= 0 || NH <= 0 || T <= 0 || DHQK <= 0 || DHHV <= 0) return "mlstm_hip_recurrent_sequence: non-positive dimension";
  if ((long long)B * NH > 65535) return "mlstm_hip_recurrent_sequence: B*NH exceeds 65535";
  if (DHQK > 1024) return "mlstm_hip_recurrent_sequence: DHQK above 1024 does not fit the register-resident state slice";
#define MLSTM_SEQ_ARGS q, k, v, i, f, c_in, n_in, m_in, h, c_out, n_out, m_out, B, NH, T, DHQK, DHHV, eps, dtype_qkv, dtype_gates, dtype_state, stream
  // rows per lane x columns per lane: at most 128 state registers per lane
  const bool vec = DHHV % 4 == 0;
#define MLSTM_SEQ_PICK(RPT_, CPT_, VEC_)                                                          \
  return dtype_qkv == 0   ? launch_step_seq_t<RPT_, CPT_, VEC_, 0>(MLSTM_SEQ_ARGS)                \
         : dtype_qkv == 1 ? launch_step_seq_t<RPT_, CPT_, VEC_, 1>(MLSTM_SEQ_ARGS)                \
                          : launch_step_seq_t<RPT_, CPT_, VEC_, 2>(MLSTM_SEQ_ARGS)
  if (DHQK <= 128) {
    if (vec) MLSTM_SEQ_PICK(16, 4, true);
    MLSTM_SEQ_PICK(16, 4, false);
  }
  if (DHQK <= 256) {
    if (vec) MLSTM_SEQ_PICK(32, 4, true);
    MLSTM_SEQ_PICK(32, 4, false);
  }
  if (DHQK <= 512) MLSTM_SEQ_PICK(64, 2, false);
  MLSTM_SEQ_PICK(128, 1, false);
#undef MLSTM_SEQ_PICK
#undef MLSTM_SEQ_ARGS
}

}  // namespace mlstm
