// Allocation-free variant of the chunkwise forward: mlstm_hip_chunkwise_fw_noalloc (declared in include/mlstm_hip.h).
//
// For callers that cannot allocate device memory around the call (code under HIP graph capture, tight serving loops,
// harnesses that forbid hipMalloc): the workspace the forward needs (gate vectors, per-chunk normaliser states, kept
// chunk states) lives in a file-scope device array owned by the library instead of a caller-provided buffer.  Every GPU
// the library runs on holds its own copy of the array until the process ends.  Host code never uses the array's name
// as an address (it is only a stand-in on the host side): the per-device address comes from hipGetSymbolAddress, looked
// up once per device with that device current, and that pointer is what the kernels and copies receive.
//
// Calls on one GPU share that GPU's array: calls that overlap in time on one GPU (different streams or threads) race.
// Nothing has to be cleared between calls: every part of the workspace is written by the kernels before it is read.
#include <hip/hip_runtime.h>
#include <stdio.h>

#include <mutex>

#include "../../include/mlstm_hip.h"
#include "kernels.h"

namespace {
static __device__ __align__(256) unsigned char scratch[MLSTM_NOALLOC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Address of `scratch` on the current device, or nullptr with *err set.
void* scratch_on_current_device(const char** err) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    *err = "cannot identify the current device";
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      *err = "hipGetSymbolAddress failed for the static scratch";
      return nullptr;
    }
    g_scratch_ptr[dev] = p;
  }
  return g_scratch_ptr[dev];
}

int fail_noalloc(const char* what) {
  char msg[256];
  snprintf(msg, sizeof(msg), "mlstm_hip_chunkwise_fw_noalloc: %s", what);
  return mlstm::set_last_error(msg);
}
}  // namespace

extern "C" int mlstm_hip_chunkwise_fw_noalloc(const void* q, const void* k, const void* v, const void* i, const void* f,
                                              const float* c0, const float* n0, const float* m0, void* H, float* n_out,
                                              float* m_out, float* c_last, float* n_last, float* m_last, int B, int NH,
                                              int S, int DHQK, int DHHV, float eps, int dtype_qkv, int dtype_gates,
                                              int gate, int normalize, void* stream) {
  const size_t need = mlstm_hip_chunkwise_fw_workspace_bytes(B, NH, S, DHQK, DHHV, /*keep_for_backward=*/0,
                                                             MLSTM_PATH_AUTO, /*state_stride=*/0);
  if (need == 0) return fail_noalloc("unsupported shape (head dimensions must be multiples of 64, DHQK <= 896, B*NH <= 65535)");
  if (need > (size_t)MLSTM_NOALLOC_SCRATCH_BYTES) {
    char msg[200];
    snprintf(msg, sizeof(msg),
             "this shape needs %zu bytes of scratch, the static scratch holds %zu; use mlstm_hip_chunkwise_fw with a "
             "caller-provided workspace",
             need, (size_t)MLSTM_NOALLOC_SCRATCH_BYTES);
    return fail_noalloc(msg);
  }
  const char* err = nullptr;
  void* ws = scratch_on_current_device(&err);
  if (ws == nullptr) return fail_noalloc(err);
  return mlstm_hip_chunkwise_fw(q, k, v, i, f, c0, n0, m0, H, n_out, m_out, c_last, n_last, m_last, ws,
                                (size_t)MLSTM_NOALLOC_SCRATCH_BYTES, /*keep_for_backward=*/0, B, NH, S, DHQK, DHHV, eps,
                                dtype_qkv, dtype_gates, gate, normalize, MLSTM_PATH_AUTO, /*state_stride=*/0,
                                MLSTM_NORM_NONE, 0.f, nullptr, nullptr, stream);
}
