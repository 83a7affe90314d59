// Host-visible launch interface of the kernel translation units (argument structs + launchers).
// Every launcher validates what its kernel's indexing assumes, enqueues on `stream`, and returns nullptr
// on success or a static message describing the rejected argument.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "layout.h"

namespace mlstm {

struct ScanArgs {
  const uint16_t* X;      // (B,NH,S,DHQK) bf16: K (forward) or Q (backward)
  const uint16_t* Y;      // (B,NH,S,DHHV) bf16: V (forward) or dH (backward)
  const float* scale_a;   // [BH][Sp] forward: abar; backward: bbar
  const float* nrow;      // backward: [BH][Sp] row normaliser or nullptr; forward: nullptr
  const float* gbar;      // [BH][NC]
  const float* init;      // (B,NH,DHQK,DHHV) fp32 or nullptr (zeros)
  uint16_t* states;       // bf16 fragments [BH][NC][DHHV/32][DHQK/16][64][8]
  float* final_out;       // (B,NH,DHQK,DHHV) fp32 or nullptr
  const float* n_init;    // forward: (B,NH,DHQK) or nullptr
  float* nstates;         // forward: [BH][NC][DHQK] or nullptr (skip the n recurrence)
  float* n_final;         // forward: (B,NH,DHQK) or nullptr
  int S, NC, DHQK, DHHV;
  float qk_scale, eps;
  int backward;
};

struct ParFwArgs {
  const uint16_t *Q, *K, *V;
  GateBufs g;
  const float* nstates;
  const uint16_t* cstates;
  float* nrow;      // workspace [BH][Sp]
  uint16_t* H;      // (B,NH,S,DHHV) bf16
  float* n_out;     // optional (B,NH,S)
  float* m_out;     // optional (B,NH,S)
  int S, NC, DHQK, DHHV;
  float qk_scale, eps;
  int sig_gate, normalize;
};

const char* launch_step(const void* q, const void* k, const void* v, const void* i, const void* f,
                        const float* c_in, const float* n_in, const float* m_in, void* h, float* c_out,
                        float* n_out, float* m_out, int B, int NH, int DHQK, int DHHV, float eps,
                        int dtype_qkv, int dtype_gates, hipStream_t stream);
const char* launch_gates(const void* i, const void* f, const float* m0, const GateBufs& gb, float* m_last,
                         int B, int NH, int S, int dtype_gates, int sig_gate, hipStream_t stream);
const char* launch_scan(const ScanArgs& a, int BH, bool hilo, hipStream_t stream);
const char* launch_par_fw(const ParFwArgs& a, int BH, hipStream_t stream);

}  // namespace mlstm
