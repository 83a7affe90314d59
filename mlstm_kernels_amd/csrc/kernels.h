// Host-visible launch interface of the kernel translation units (argument structs + launchers).
// Every launcher validates what its kernel's indexing assumes, enqueues on `stream`, and returns nullptr
// on success or a static message describing the rejected argument.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "layout.h"

namespace mlstm {

struct ScanArgs {
  const uint16_t* X;      // (B,NH,S,DHQK) bf16/fp16: K (forward) or Q (backward)
  const uint16_t* Y;      // (B,NH,S,DHHV) bf16/fp16: V (forward) or dH (backward)
  const float* scale_a;   // [BH][Sp] forward: abar; backward: bbar
  const float* nrow;      // backward: [BH][Sp] row normaliser or nullptr; forward: nullptr
  const float* gbar;      // [BH][NC]
  const float* init;      // (B,NH,DHQK,DHHV) fp32 or nullptr (zeros)
  uint16_t* states;       // bf16 fragments [BH][ceil(NC/stride)][DHHV/32][DHQK/16][64][8]
  float* final_out;       // (B,NH,DHQK,DHHV) fp32 or nullptr
  const float* n_init;    // forward: (B,NH,DHQK) or nullptr
  float* nstates;         // forward: [BH][NC][3][DHQK] (three partial vectors per chunk) or nullptr (skip the n recurrence)
  float* n_final;         // forward: (B,NH,DHQK) or nullptr
  int S, NC, DHQK, DHHV;
  float qk_scale, eps;
  int backward;
  int stride;             // a chunk state is kept every `stride` chunks
  int f16;                // X, Y and the state fragments are float16 instead of bfloat16
  int all_remainder;      // forward, last state returned: every chunk carries the remainder of the value operand (the
                          // sigmoid input gate has no stabiliser, so the decay factors alone do not say which chunks
                          // still weigh in the last state)
  int part;               // set by the launcher: 0 whole sequence; 1 / 2 the two launches of a forward scan that
                          // returns the last state (before / from the first chunk that carries the remainder)
};

struct ParHvArgs {
  const uint16_t *Q, *K, *V, *dH;  // forward uses Q,K,V; dV uses Q,K,dH
  GateBufs g;
  const float* nstates;     // forward: n before each chunk, [BH][NC][3][DHQK]: three partial vectors to add up
  const uint16_t* states;   // forward: C states; dV: dC states
  const float* nrow;        // dV: row normaliser (input)
  float* nrow_out;          // forward: row normaliser (output, workspace [BH][Sp])
  uint16_t* Out;            // (B,NH,S,DHHV) bf16: H or dV
  float* n_out;             // forward, optional (B,NH,S)
  float* m_out;             // forward, optional (B,NH,S)
  int S, NC, DHQK, DHHV;
  float qk_scale, eps;
  int sig_gate;
  int use_nrow;             // 0 only for the un-normalised sigmoid-gate variant
  int stride;               // a chunk state is kept every `stride` chunks
  int head_norm;            // forward: 0 none, 1 layer norm, 2 rms norm over the DHHV columns of every row of H
  float norm_eps;
  float* norm_mean;         // forward with head_norm: (B,NH,S) row means (0 for rms)
  float* norm_rstd;         // forward with head_norm: (B,NH,S) reciprocal standard deviations
  int f16;                  // inputs, state fragments and Out are float16 instead of bfloat16
};

struct HeadNormBwArgs {
  const uint16_t* dY;       // (rows, D) bf16 gradient of the normalised output
  const uint16_t* Y;        // (rows, D) bf16 normalised output
  const float* rstd;        // (rows)
  uint16_t* dX;             // (rows, D) bf16 gradient of the input of the norm
  size_t rows;
  int D, kind;              // kind: 1 layer norm, 2 rms norm
  int f16;                  // dY, Y and dX are float16 instead of bfloat16
};

struct FusedHvArgs {
  const uint16_t *Q, *K, *V, *dH;  // forward uses Q,K,V; dV uses Q,K,dH
  GateBufs g;
  const float* init;        // (B,NH,DHQK,DHHV) fp32 initial state (forward: C0, dV: dC_last) or nullptr (zeros)
  const float* n_init;      // forward: (B,NH,DHQK) or nullptr
  const float* nrow;        // dV: row normaliser of the forward pass
  uint16_t* states;         // bf16 state fragments [BH][ceil(NC/stride)][DHHV/32][DHQK/16][64][8] or nullptr (not emitted)
  uint16_t* Out;            // (B,NH,S,DHHV) bf16: H or dV
  float* nrow_out;          // forward: row normaliser (workspace [BH][Sp])
  float* n_out;             // forward, optional (B,NH,S)
  float* m_out;             // forward, optional (B,NH,S)
  float* final_out;         // (B,NH,DHQK,DHHV) fp32 or nullptr: C_last (forward) / dC0 (dV)
  float* n_final;           // forward: (B,NH,DHQK) or nullptr
  int S, NC, DHQK, DHHV;
  float qk_scale, eps;
  int sig_gate;
  int use_nrow;             // 0 only for the un-normalised sigmoid-gate variant (n is then not tracked)
  int stride;               // a chunk state is emitted every `stride` chunks
};

struct ParQkArgs {
  const uint16_t *Q, *K, *V, *dH;
  GateBufs g;
  const uint16_t* states;   // dQ: C states; dK: dC states
  const float* nrow;
  uint16_t* Out;            // (B,NH,S,DHQK) bf16: dQ or dK
  float* rowdot;            // [DHQK tiles][BH][Sp]: sum_d q*dQ (dQ) or sum_d k*dK (dK) over the rows of one tile
  const uint16_t* states2;  // the dK operands (dC states, dK, sum_d k*dK); states, Out and rowdot above are the
  uint16_t* Out2;           // dQ operands
  float* rowdot2;
  int S, NC, DHQK, DHHV;
  float qk_scale, eps;
  int use_nrow;
  int stride;               // a chunk state is kept every `stride` chunks
  int f16;                  // inputs, state fragments and outputs are float16 instead of bfloat16
};

struct GateGradArgs {
  const void *i, *f;        // gate pre-activations (B,NH,S)
  const float *qdq, *kdk;   // [ntiles][BH][Sp]: one slot per head-dimension tile of the dQ/dK kernel
  int ntiles;
  float *dI, *dF;           // (B,NH,S) fp32
  int S, NC, dtype_gates, sig_gate;
};

const char* launch_step(const void* q, const void* k, const void* v, const void* i, const void* f,
                        const void* c_in, const void* n_in, const void* m_in, void* h, void* c_out,
                        void* n_out, void* m_out, int B, int NH, int DHQK, int DHHV, float eps,
                        int dtype_qkv, int dtype_gates, int dtype_state, hipStream_t stream);
const char* launch_step_seq(const void* q, const void* k, const void* v, const void* i, const void* f,
                            const void* c_in, const void* n_in, const void* m_in, void* h, void* c_out,
                            void* n_out, void* m_out, int B, int NH, int T, int DHQK, int DHHV, float eps,
                            int dtype_qkv, int dtype_gates, int dtype_state, hipStream_t stream);
const char* launch_gates(const void* i, const void* f, const float* m0, const GateBufs& gb, float* m_last,
                         int B, int NH, int S, int dtype_gates, int sig_gate, hipStream_t stream);
const char* launch_scan(const ScanArgs& a, int BH, bool hilo, hipStream_t stream);
const char* launch_par_hv(const ParHvArgs& a, int BH, bool is_dv, hipStream_t stream);
bool par_hv_head_norm_supported(int DHHV);
// streaming (persistent, producer / consumer waves) form of the same two kernels for the shapes it supports
bool stream_hv_supported(const ParHvArgs& a);
const char* launch_stream_hv(const ParHvArgs& a, int BH, bool is_dv, hipStream_t stream);
const char* launch_head_norm_bw(const HeadNormBwArgs& a, hipStream_t stream);
bool fused_hv_supported(int DHQK, int DHHV);
const char* launch_fused_hv(const FusedHvArgs& a, int BH, bool is_dv, hipStream_t stream);
const char* launch_par_qk_pair(const ParQkArgs& a, int BH, hipStream_t stream);
// streaming (persistent, producer / consumer waves) form of the same launch for the shapes it supports
bool window_qk_supported(const ParQkArgs& a);
const char* launch_window_qk(const ParQkArgs& a, int BH, hipStream_t stream);
bool stream_qk_supported(const ParQkArgs& a);
const char* launch_stream_qk(const ParQkArgs& a, int BH, hipStream_t stream);
int par_qk_head_tile(int DHQK);  // head-dimension rows per workgroup of the dQ/dK kernel
const char* launch_gate_grads(const GateGradArgs& a, int BH, hipStream_t stream);
const char* launch_fill_zero(float* p, size_t n, hipStream_t stream);
// stores `msg` as the calling thread's last error (what mlstm_hip_last_error returns) and returns 1
int set_last_error(const char* msg);

}  // namespace mlstm
