// Memory layout of the caller-provided workspaces (host and device views).
//
// Forward workspace (everything the backward re-uses lives here):
//   gate vectors   u, w, abar, bbar, mcomb     5 x fp32 [B*NH][NC*128]
//   per chunk      gbar, amax, graw            3 x fp32 [B*NH][NC]
//   stabiliser     mstates                     fp32 [B*NH][NC+1]   (index c = value before chunk c)
//   normaliser     nstates                     fp32 [B*NH][NC][3][DHQK] (n before chunk c, as three partial vectors
//                                              to be added up: the scan accumulates them on the matrix cores)
//   row normaliser nrow                        fp32 [B*NH][NC*128]  max(|den|, floor), without eps
//   chunk states   cstates                     bf16 [B*NH][ceil(NC/stride)][DHHV/32][DHQK/16][64 lanes][8]
//                  (the state before every stride-th chunk; stride 1 keeps all of them)
//
// A chunk state is stored as ready-made MFMA operand fragments of C^T: fragment (wb, ds) holds, for lane
// l = 32*h + r and element e, the value C[16*ds + 8*(e/4) + 4*h + e%4][32*wb + r].  That is exactly how the
// 32x32 accumulator tiles of the scan kernel hold C (4 consecutive rows per register group), so the scan
// stores 16 B per lane fully coalesced, and the consumers load 16 B per lane straight into an A operand
// (the permutation of the 16 rows inside a fragment is irrelevant to a contraction over them as long as
// the other operand uses the same order).
#pragma once
#include <stddef.h>
#include <stdint.h>

namespace mlstm {

constexpr int kMaxStateStride = 8;  // chunk states are kept every 1 .. 8 chunks

struct GateBufs {
  float *u, *w, *abar, *bbar, *mcomb, *gbar, *amax, *mstates;
  float* graw;  // per chunk: sum of logsig(f) over the chunk (input of the scan over chunks that yields gbar)
};

struct FwWorkspace {
  GateBufs g;
  float* nstates;
  float* nrow;
  uint16_t* cstates;
  size_t bytes;
};

struct BwWorkspace {
  uint16_t* dcstates;  // same fragment layout as cstates; slot s = gradient of the state after the last chunk of group s
  float* qdq;          // fp32 [tiles][B*NH][NC*128]: sum_d q*dQ per position and head-dimension tile
  float* kdk;          // fp32 [tiles][B*NH][NC*128]: sum_d k*dK per position and head-dimension tile
  size_t bytes;
};

inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

// with_states = false leaves out the chunk states (forward passes whose states nobody reads: cstates is null)
inline FwWorkspace carve_fw_workspace(void* base, int B, int NH, int S, int DHQK, int DHHV, bool with_states,
                                      int stride) {
  const size_t BH = (size_t)B * NH, NC = (size_t)(S + 127) / 128, Sp = NC * 128;
  const size_t NCS = (NC + stride - 1) / stride;
  char* p = (char*)base;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    char* r = p + off;
    off += align256(bytes);
    return r;
  };
  FwWorkspace w;
  w.g.u = (float*)take(BH * Sp * 4);
  w.g.w = (float*)take(BH * Sp * 4);
  w.g.abar = (float*)take(BH * Sp * 4);
  w.g.bbar = (float*)take(BH * Sp * 4);
  w.g.mcomb = (float*)take(BH * Sp * 4);
  w.g.gbar = (float*)take(BH * NC * 4);
  w.g.amax = (float*)take(BH * NC * 4);
  w.g.mstates = (float*)take(BH * (NC + 1) * 4);
  w.g.graw = (float*)take(BH * NC * 4);
  w.nstates = (float*)take(BH * NC * 3 * DHQK * 4);
  w.nrow = (float*)take(BH * Sp * 4);
  w.cstates = with_states ? (uint16_t*)take(BH * NCS * (size_t)DHQK * DHHV * 2) : nullptr;
  w.bytes = off;
  return w;
}

inline BwWorkspace carve_bw_workspace(void* base, int B, int NH, int S, int DHQK, int DHHV, int stride, int tiles) {
  const size_t BH = (size_t)B * NH, NC = (size_t)(S + 127) / 128, Sp = NC * 128;
  const size_t NCS = (NC + stride - 1) / stride;
  char* p = (char*)base;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    char* r = p + off;
    off += align256(bytes);
    return r;
  };
  BwWorkspace w;
  w.dcstates = (uint16_t*)take(BH * NCS * (size_t)DHQK * DHHV * 2);
  w.qdq = (float*)take((size_t)tiles * BH * Sp * 4);
  w.kdk = (float*)take((size_t)tiles * BH * Sp * 4);
  w.bytes = off;
  return w;
}

}  // namespace mlstm
