// C ABI of libmlstm_hip.so (declared in include/mlstm_hip.h): argument validation, workspace carving and
// kernel sequencing.  No device memory is allocated here and no state is kept between calls (kernel path and state
// stride are per-call arguments).
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/mlstm_hip.h"
#include "kernels.h"

namespace {
thread_local char g_err[512] = "";

// Optional per-kernel timing: when enabled, every kernel launch issued by this library is bracketed by a
// pair of HIP events recorded on the launch stream.  Host-side bookkeeping only; no device memory.
struct TimedLaunch {
  const char* name;
  hipEvent_t start, stop;
};
std::mutex g_prof_mutex;
std::atomic<bool> g_prof_on{false};   // read by every launch, written by mlstm_profile_enable from any thread
std::vector<TimedLaunch> g_prof_launches;

struct ProfileScope {
  const char* name;
  hipStream_t stream;
  hipEvent_t start = nullptr, stop = nullptr;
  bool active = false;
  ProfileScope(const char* n, hipStream_t s) : name(n), stream(s) {
    if (!g_prof_on.load(std::memory_order_relaxed)) return;
    if (hipEventCreate(&start) != hipSuccess || hipEventCreate(&stop) != hipSuccess) return;
    active = true;
    (void)hipEventRecord(start, stream);
  }
  ~ProfileScope() {
    if (!active) return;
    (void)hipEventRecord(stop, stream);
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    g_prof_launches.push_back({name, start, stop});
  }
};
int fail(const char* msg) {
  snprintf(g_err, sizeof(g_err), "%s", msg);
  return 1;
}
int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(e));
    return 1;
  }
  return 0;
}
// Which kernels carry the value-column side of the chunkwise passes (H forward, dV backward):
//   split : state scan, then a chunk-parallel kernel reading the materialised chunk states
//   fused : one sequential kernel per pass that keeps the state slice in registers
// The fused kernels move far fewer bytes (no chunk state is written or re-read by them) but run one four-wave
// workgroup per (batch, head, 64 value columns) and per CU, which leaves them latency-bound: on MI355X at
// B*S = 65536, NH = 8, 256/512 the fused forward is about twice as slow as scan + streaming kernel.  Opt-in only.
bool use_fused(int path, int DHQK, int DHHV) { return path == MLSTM_PATH_FUSED && mlstm::fused_hv_supported(DHQK, DHHV); }
// Chunk states are kept every `stride` chunks of 128 positions (0 = the default for the shape).  Fewer kept states
// mean less HBM traffic (a state is DHQK x DHHV bf16 per chunk and head, written once and read by three kernels)
// against more score blocks in the chunk-parallel kernels.
constexpr int kDefaultStateStride = 2;
int resolve_stride(int state_stride) { return state_stride == 0 ? kDefaultStateStride : state_stride; }
const char* check_options(int path, int state_stride, int DHQK, int DHHV) {
  if (path != MLSTM_PATH_AUTO && path != MLSTM_PATH_SPLIT && path != MLSTM_PATH_FUSED && path != MLSTM_PATH_STREAM)
    return "unknown kernel path code";
  if (path == MLSTM_PATH_FUSED && !mlstm::fused_hv_supported(DHQK, DHHV))
    return "the fused kernel path supports DHQK = 128 or 256 only";
  if (state_stride < 0 || state_stride > mlstm::kMaxStateStride) return "state_stride must be 0 (default) or 1 .. 8";
  return nullptr;
}
// H / dV kernel of the split form: the streaming kernel where the path asks for it (or leaves the choice open) and the
// shape is one it supports, otherwise the tiled kernel
const char* launch_hv(int path, const mlstm::ParHvArgs& a, int BH, bool is_dv, hipStream_t st) {
  if (path == MLSTM_PATH_STREAM && !mlstm::stream_hv_supported(a))
    return "the stream kernel path supports DHQK = 256, DHHV % 512 == 0, S % 128 == 0 only (with a head norm: DHHV = 512)";
  if ((path == MLSTM_PATH_STREAM || path == MLSTM_PATH_AUTO) && mlstm::stream_hv_supported(a))
    return mlstm::launch_stream_hv(a, BH, is_dv, st);
  return mlstm::launch_par_hv(a, BH, is_dv, st);
}
// dQ / dK launch.  MLSTM_PATH_STREAM: the window kernel (state stride 2) or the streaming kernel per chunk and
// gradient (other strides); MLSTM_PATH_AUTO: the window kernel where the shape allows, else the tiled pair kernel
// (faster than the per-chunk streaming kernel); MLSTM_PATH_SPLIT: the tiled pair kernel
const char* launch_qk(int path, const mlstm::ParQkArgs& a, int BH, hipStream_t st) {
  if (path == MLSTM_PATH_STREAM && !mlstm::stream_qk_supported(a))
    return "the stream kernel path supports DHQK = 256, DHHV % 512 == 0, S % 128 == 0 only (with a head norm: DHHV = 512)";
  if ((path == MLSTM_PATH_STREAM || path == MLSTM_PATH_AUTO) && mlstm::window_qk_supported(a))
    return mlstm::launch_window_qk(a, BH, st);
  if (path == MLSTM_PATH_STREAM) return mlstm::launch_stream_qk(a, BH, st);
  return mlstm::launch_par_qk_pair(a, BH, st);
}
const char* check_dims(int B, int NH, int S, int DHQK, int DHHV) {
  if (B <= 0 || NH <= 0 || S <= 0) return "B, NH and S must be positive";
  if (DHQK <= 0 || DHHV <= 0 || DHQK % 64 != 0 || DHHV % 64 != 0) return "DHQK and DHHV must be positive multiples of 64";
  if ((long long)B * NH > 65535) return "B*NH exceeds 65535";
  // the chunk-parallel kernels keep 64 rows of q or k resident in LDS (132 bytes per head-dimension entry beside
  // 40 KB of tiles, 160 KB per workgroup at most)
  if (DHQK > 896) return "DHQK too large for the LDS-resident tile (at most 896)";
  return nullptr;
}
}  // namespace

namespace mlstm {
int set_last_error(const char* msg) { return fail(msg); }
}  // namespace mlstm

static bool valid_dtype(int code) { return code == MLSTM_F32 || code == MLSTM_BF16 || code == MLSTM_F16; }

extern "C" {

int mlstm_hip_abi_version(void) { return 6; }

int mlstm_hip_profile_enable(int on) {
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  g_prof_on.store(on != 0, std::memory_order_relaxed);
  return 0;
}

int mlstm_hip_profile_read(int index, char* name, size_t name_cap, float* total_ms, int* launches) {
  // Aggregates the recorded launches by kernel name (first call of a read-out pass: index 0), waits for their
  // events, and returns the number of distinct kernels; entry `index` is copied out when it exists.
  static std::vector<std::string> names;
  static std::vector<float> totals;
  static std::vector<int> counts;
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  if (index == 0) {
    names.clear(); totals.clear(); counts.clear();
    for (TimedLaunch& t : g_prof_launches) {
      float ms = 0.f;
      if (hipEventSynchronize(t.stop) == hipSuccess) (void)hipEventElapsedTime(&ms, t.start, t.stop);
      (void)hipEventDestroy(t.start);
      (void)hipEventDestroy(t.stop);
      size_t k = 0;
      for (; k < names.size(); ++k)
        if (names[k] == t.name) break;
      if (k == names.size()) { names.push_back(t.name); totals.push_back(0.f); counts.push_back(0); }
      totals[k] += ms;
      counts[k] += 1;
    }
    g_prof_launches.clear();
  }
  if (index >= 0 && (size_t)index < names.size()) {
    if (name && name_cap) snprintf(name, name_cap, "%s", names[index].c_str());
    if (total_ms) *total_ms = totals[index];
    if (launches) *launches = counts[index];
  }
  return (int)names.size();
}
const char* mlstm_hip_last_error(void) { return g_err; }

int mlstm_hip_step(const void* q, const void* k, const void* v, const void* i, const void* f, const void* c_in,
                   const void* n_in, const void* m_in, void* h, void* c_out, void* n_out, void* m_out, int B, int NH,
                   int DHQK, int DHHV, float eps, int dtype_qkv, int dtype_gates, int dtype_state, void* stream) {
  if (!q || !k || !v || !i || !f || !c_in || !n_in || !m_in || !h || !c_out || !n_out || !m_out)
    return fail("mlstm_hip_step: null pointer argument");
  if (n_out == n_in || m_out == m_in)
    return fail("mlstm_hip_step: n_out/m_out must not alias n_in/m_in (only C may be updated in place)");
  if (!valid_dtype(dtype_qkv) || !valid_dtype(dtype_gates) || !valid_dtype(dtype_state))
    return fail("mlstm_hip_step: unsupported dtype code");
  {
    ProfileScope ps("step", (hipStream_t)stream);
    const char* e = mlstm::launch_step(q, k, v, i, f, c_in, n_in, m_in, h, c_out, n_out, m_out, B, NH, DHQK, DHHV, eps,
                                       dtype_qkv, dtype_gates, dtype_state, (hipStream_t)stream);
    if (e) return fail(e);
  }
  return check_launch("mlstm_hip_step");
}

int mlstm_hip_recurrent_sequence(const void* q, const void* k, const void* v, const void* i, const void* f,
                                 const void* c_in, const void* n_in, const void* m_in, void* h, void* c_out,
                                 void* n_out, void* m_out, int B, int NH, int T, int DHQK, int DHHV, float eps,
                                 int dtype_qkv, int dtype_gates, int dtype_state, void* stream) {
  if (!q || !k || !v || !i || !f || !c_in || !n_in || !m_in || !h || !c_out || !n_out || !m_out)
    return fail("mlstm_hip_recurrent_sequence: null pointer argument");
  if (n_out == n_in || m_out == m_in)
    return fail("mlstm_hip_recurrent_sequence: n_out/m_out must not alias n_in/m_in (only C may be updated in place)");
  if (!valid_dtype(dtype_qkv) || !valid_dtype(dtype_gates) || !valid_dtype(dtype_state))
    return fail("mlstm_hip_recurrent_sequence: unsupported dtype code");
  {
    ProfileScope ps("step_seq", (hipStream_t)stream);
    const char* e = mlstm::launch_step_seq(q, k, v, i, f, c_in, n_in, m_in, h, c_out, n_out, m_out, B, NH, T, DHQK, DHHV,
                                           eps, dtype_qkv, dtype_gates, dtype_state, (hipStream_t)stream);
    if (e) return fail(e);
  }
  return check_launch("mlstm_hip_recurrent_sequence");
}

size_t mlstm_hip_chunkwise_fw_workspace_bytes(int B, int NH, int S, int DHQK, int DHHV, int keep_for_backward, int path,
                                              int state_stride) {
  if (check_dims(B, NH, S, DHQK, DHHV) || check_options(path, state_stride, DHQK, DHHV)) return 0;
  const bool with_states = keep_for_backward || !use_fused(path, DHQK, DHHV);
  return mlstm::carve_fw_workspace(nullptr, B, NH, S, DHQK, DHHV, with_states, resolve_stride(state_stride)).bytes;
}

}  // extern "C"

namespace {
// The forward pass proper: arguments validated, workspace carved from `workspace`.
int chunkwise_fw_impl(const char* who, const void* q, const void* k, const void* v, const void* i, const void* f,
                      const float* c0, const float* n0, const float* m0, void* H, float* n_out, float* m_out,
                      float* c_last, float* n_last, float* m_last, void* workspace, size_t workspace_bytes,
                      int keep_for_backward, int B, int NH, int S, int DHQK, int DHHV, float eps, int dtype_qkv,
                      int dtype_gates, int gate, int normalize, int path, int state_stride, int head_norm,
                      float norm_eps, float* norm_mean, float* norm_rstd, hipStream_t st) {
  char msg[160];
  auto failw = [&](const char* what) {
    snprintf(msg, sizeof(msg), "%s: %s", who, what);
    return fail(msg);
  };
  if (!q || !k || !v || !i || !f || !H || !workspace) return failw("null pointer argument");
  if (const char* e = check_dims(B, NH, S, DHQK, DHHV)) return failw(e);
  if (const char* e = check_options(path, state_stride, DHQK, DHHV)) return failw(e);
  if (dtype_qkv != MLSTM_BF16 && dtype_qkv != MLSTM_F16) return failw("q/k/v must be bf16 or fp16");
  if (dtype_gates != MLSTM_F32 && dtype_gates != MLSTM_BF16 && dtype_gates != MLSTM_F16) return failw("unsupported gate dtype");
  const int f16 = dtype_qkv == MLSTM_F16;
  if (gate != MLSTM_GATE_EXP && gate != MLSTM_GATE_SIG) return failw("unknown gate code");
  const bool has_c0 = c0 != nullptr;
  if (has_c0 != (n0 != nullptr)) return failw("c0 and n0 must be given together");
  if (gate == MLSTM_GATE_EXP && has_c0 != (m0 != nullptr)) return failw("initial states must be given together");
  const bool fused = use_fused(path, DHQK, DHHV);
  if (fused && f16) return failw("the fused kernel path multiplies bf16 operands only");
  if (head_norm != MLSTM_NORM_NONE) {
    if (head_norm != MLSTM_NORM_LAYER && head_norm != MLSTM_NORM_RMS) return failw("unknown head norm code");
    if (fused) return failw("the fused kernel path has no head norm epilogue");
    if (!mlstm::par_hv_head_norm_supported(DHHV)) return failw("the fused head norm needs DHHV = 64, 128, 256 or 512");
    if (!norm_mean || !norm_rstd) return failw("the head norm needs its mean and rstd outputs");
  }
  const bool with_states = keep_for_backward || !fused;
  const int stride = resolve_stride(state_stride);
  mlstm::FwWorkspace ws = mlstm::carve_fw_workspace(workspace, B, NH, S, DHQK, DHHV, with_states, stride);
  if (workspace_bytes < ws.bytes) return failw("workspace too small");
  const int NC = (S + 127) / 128, BH = B * NH;
  const int sig = gate == MLSTM_GATE_SIG;
  {
    ProfileScope ps("gates", st);
    if (const char* e = mlstm::launch_gates(i, f, m0, ws.g, m_last, B, NH, S, dtype_gates, sig, st)) return fail(e);
  }
  if (check_launch("gates")) return 1;

  const bool track_n = !(sig && !normalize);  // the un-normalised sigmoid-gate variant leaves n untouched
  if (!track_n && n_last != nullptr) {
    if (n0 != nullptr) {
      if (hipMemcpyAsync(n_last, n0, (size_t)BH * DHQK * sizeof(float), hipMemcpyDeviceToDevice, st) != hipSuccess)
        return failw("copying n0 to n_last failed");
    } else if (const char* e = mlstm::launch_fill_zero(n_last, (size_t)BH * DHQK, st)) {
      return fail(e);
    }
  }
  if (fused) {
    mlstm::FusedHvArgs fa;
    memset(&fa, 0, sizeof(fa));
    fa.Q = (const uint16_t*)q; fa.K = (const uint16_t*)k; fa.V = (const uint16_t*)v;
    fa.g = ws.g;
    fa.init = c0;
    fa.n_init = n0;
    fa.states = keep_for_backward ? ws.cstates : nullptr;
    fa.Out = (uint16_t*)H;
    fa.nrow_out = ws.nrow;
    fa.n_out = n_out; fa.m_out = m_out;
    fa.final_out = c_last;
    fa.n_final = track_n ? n_last : nullptr;
    fa.S = S; fa.NC = NC; fa.DHQK = DHQK; fa.DHHV = DHHV;
    fa.qk_scale = 1.0f / sqrtf((float)DHQK);
    fa.eps = eps;
    fa.sig_gate = sig;
    fa.use_nrow = track_n;
    fa.stride = stride;
    {
      ProfileScope ps("fused_fw", st);
      if (const char* e = mlstm::launch_fused_hv(fa, BH, /*is_dv=*/false, st)) return fail(e);
    }
    return check_launch("fused_hv forward");
  }

  mlstm::ScanArgs sa;
  memset(&sa, 0, sizeof(sa));
  sa.X = (const uint16_t*)k;
  sa.Y = (const uint16_t*)v;
  sa.scale_a = ws.g.abar;
  sa.gbar = ws.g.gbar;
  sa.init = c0;
  sa.states = ws.cstates;
  sa.final_out = c_last;
  sa.n_init = n0;
  sa.nstates = track_n ? ws.nstates : nullptr;
  sa.n_final = track_n ? n_last : nullptr;
  sa.S = S; sa.NC = NC; sa.DHQK = DHQK; sa.DHHV = DHHV;
  sa.qk_scale = 1.0f / sqrtf((float)DHQK);
  sa.eps = eps;
  sa.backward = 0;
  sa.stride = stride;
  sa.f16 = f16;
  // Which chunks still weigh in the last state is read off the decay factors, which presumes inputs of comparable
  // scale in every chunk: true for the exponential gate (its stabiliser rescales them), not for the sigmoid gate,
  // whose late positions may all be closed while early chunks dominate the state.
  sa.all_remainder = sig;
  {
    ProfileScope ps("scan_fw", st);
    // The head + remainder split of the value operand only serves the fp32 last state (1e-5 instead of 1.5e-3
    // relative); the chunk states are rounded to 16 bits anyway, so a call that returns no last state skips it.
    if (const char* e = mlstm::launch_scan(sa, BH, /*hilo=*/c_last != nullptr, st)) return fail(e);
  }
  if (check_launch("scan_fw")) return 1;

  mlstm::ParHvArgs pa;
  memset(&pa, 0, sizeof(pa));
  pa.Q = (const uint16_t*)q; pa.K = (const uint16_t*)k; pa.V = (const uint16_t*)v;
  pa.g = ws.g;
  pa.nstates = ws.nstates;
  pa.states = ws.cstates;
  pa.nrow_out = ws.nrow;
  pa.Out = (uint16_t*)H;
  pa.n_out = n_out; pa.m_out = m_out;
  pa.S = S; pa.NC = NC; pa.DHQK = DHQK; pa.DHHV = DHHV;
  pa.qk_scale = sa.qk_scale; pa.eps = eps;
  pa.sig_gate = sig;
  pa.use_nrow = !(sig && !normalize);
  pa.stride = stride;
  pa.head_norm = head_norm;
  pa.f16 = f16;
  pa.norm_eps = norm_eps;
  pa.norm_mean = norm_mean;
  pa.norm_rstd = norm_rstd;
  {
    ProfileScope ps("par_h", st);
    if (const char* e = launch_hv(path, pa, BH, /*is_dv=*/false, st)) return fail(e);
  }
  return check_launch("par_hv forward");
}

}  // namespace

extern "C" {

int mlstm_hip_chunkwise_fw(const void* q, const void* k, const void* v, const void* i, const void* f, const float* c0,
                           const float* n0, const float* m0, void* H, float* n_out, float* m_out, float* c_last,
                           float* n_last, float* m_last, void* workspace, size_t workspace_bytes,
                           int keep_for_backward, int B, int NH, int S, int DHQK, int DHHV, float eps, int dtype_qkv,
                           int dtype_gates, int gate, int normalize, int path, int state_stride, int head_norm,
                           float norm_eps, float* norm_mean, float* norm_rstd, void* stream) {
  return chunkwise_fw_impl("mlstm_hip_chunkwise_fw", q, k, v, i, f, c0, n0, m0, H, n_out, m_out, c_last, n_last, m_last,
                           workspace, workspace_bytes, keep_for_backward, B, NH, S, DHQK, DHHV, eps, dtype_qkv,
                           dtype_gates, gate, normalize, path, state_stride, head_norm, norm_eps, norm_mean, norm_rstd,
                           (hipStream_t)stream);
}

size_t mlstm_hip_chunkwise_fw_saved_bytes(int B, int NH, int S, int DHQK, int DHHV) {
  if (check_dims(B, NH, S, DHQK, DHHV)) return 0;
  // the chunk states are carved last: without them the workspace is exactly the part in front of them
  return mlstm::carve_fw_workspace(nullptr, B, NH, S, DHQK, DHHV, /*with_states=*/false, 1).bytes;
}

int mlstm_hip_chunkwise_recompute_states(const void* k, const void* v, const float* c0, void* workspace,
                                         size_t workspace_bytes, int B, int NH, int S, int DHQK, int DHHV,
                                         int dtype_qkv, int state_stride, void* stream) {
  if (!k || !v || !workspace) return fail("mlstm_hip_chunkwise_recompute_states: null pointer argument");
  if (const char* e = check_dims(B, NH, S, DHQK, DHHV)) return fail(e);
  if (const char* e = check_options(MLSTM_PATH_AUTO, state_stride, DHQK, DHHV)) return fail(e);
  if (dtype_qkv != MLSTM_BF16 && dtype_qkv != MLSTM_F16)
    return fail("mlstm_hip_chunkwise_recompute_states: k/v must be bf16 or fp16");
  const int stride = resolve_stride(state_stride);
  mlstm::FwWorkspace ws = mlstm::carve_fw_workspace(workspace, B, NH, S, DHQK, DHHV, true, stride);
  if (workspace_bytes < ws.bytes) return fail("mlstm_hip_chunkwise_recompute_states: workspace too small");
  hipStream_t st = (hipStream_t)stream;
  mlstm::ScanArgs sa;
  memset(&sa, 0, sizeof(sa));
  sa.X = (const uint16_t*)k;
  sa.Y = (const uint16_t*)v;
  sa.scale_a = ws.g.abar;
  sa.gbar = ws.g.gbar;
  sa.init = c0;
  sa.states = ws.cstates;
  // the normaliser states in front of the chunk states are the forward's own: the recurrence of n is not run again
  sa.S = S; sa.NC = (S + 127) / 128; sa.DHQK = DHQK; sa.DHHV = DHHV;
  sa.qk_scale = 1.0f / sqrtf((float)DHQK);
  sa.backward = 0;
  sa.stride = stride;
  sa.f16 = dtype_qkv == MLSTM_F16;
  {
    ProfileScope ps("scan_fw_recompute", st);
    if (const char* e = mlstm::launch_scan(sa, B * NH, /*hilo=*/false, st)) return fail(e);
  }
  return check_launch("mlstm_hip_chunkwise_recompute_states");
}

int mlstm_hip_head_norm_bw(const void* dY, const void* Y, const float* rstd, void* dX, size_t rows, int D, int head_norm,
                           int dtype, void* stream) {
  if (!dY || !Y || !rstd || !dX) return fail("mlstm_hip_head_norm_bw: null pointer argument");
  if (dtype != MLSTM_BF16 && dtype != MLSTM_F16) return fail("mlstm_hip_head_norm_bw: rows must be bf16 or fp16");
  mlstm::HeadNormBwArgs a;
  a.dY = (const uint16_t*)dY; a.Y = (const uint16_t*)Y; a.rstd = rstd; a.dX = (uint16_t*)dX;
  a.rows = rows; a.D = D; a.kind = head_norm;
  a.f16 = dtype == MLSTM_F16;
  {
    ProfileScope ps("head_norm_bw", (hipStream_t)stream);
    if (const char* e = mlstm::launch_head_norm_bw(a, (hipStream_t)stream)) return fail(e);
  }
  return check_launch("mlstm_hip_head_norm_bw");
}

size_t mlstm_hip_chunkwise_bw_workspace_bytes(int B, int NH, int S, int DHQK, int DHHV, int state_stride) {
  if (check_dims(B, NH, S, DHQK, DHHV) || check_options(MLSTM_PATH_AUTO, state_stride, DHQK, DHHV)) return 0;
  return mlstm::carve_bw_workspace(nullptr, B, NH, S, DHQK, DHHV, resolve_stride(state_stride),
                                   DHQK / mlstm::par_qk_head_tile(DHQK)).bytes;
}

int mlstm_hip_chunkwise_bw(const void* q, const void* k, const void* v, const void* i, const void* f, const void* dH,
                           const float* dC_last, void* dQ, void* dK, void* dV, float* dI, float* dF, float* dC0,
                           const void* fw_workspace, size_t fw_workspace_bytes, void* bw_workspace,
                           size_t bw_workspace_bytes, int B, int NH, int S, int DHQK, int DHHV, float eps,
                           int dtype_qkv, int dtype_gates, int gate, int normalize, int path, int state_stride,
                           void* stream) {
  if (!q || !k || !v || !i || !f || !dH || !dQ || !dK || !dV || !dI || !dF || !fw_workspace || !bw_workspace)
    return fail("mlstm_hip_chunkwise_bw: null pointer argument");
  if (const char* e = check_dims(B, NH, S, DHQK, DHHV)) return fail(e);
  if (const char* e = check_options(path, state_stride, DHQK, DHHV)) return fail(e);
  if (dtype_qkv != MLSTM_BF16 && dtype_qkv != MLSTM_F16) return fail("mlstm_hip_chunkwise_bw: q/k/v/dH must be bf16 or fp16");
  if (dtype_gates != MLSTM_F32 && dtype_gates != MLSTM_BF16 && dtype_gates != MLSTM_F16)
    return fail("mlstm_hip_chunkwise_bw: unsupported gate dtype");
  const int f16 = dtype_qkv == MLSTM_F16;
  if (gate != MLSTM_GATE_EXP && gate != MLSTM_GATE_SIG) return fail("mlstm_hip_chunkwise_bw: unknown gate code");
  const int stride = resolve_stride(state_stride);
  const int tiles = DHQK / mlstm::par_qk_head_tile(DHQK);
  mlstm::FwWorkspace ws = mlstm::carve_fw_workspace(const_cast<void*>(fw_workspace), B, NH, S, DHQK, DHHV, true, stride);
  if (fw_workspace_bytes < ws.bytes) return fail("mlstm_hip_chunkwise_bw: forward workspace too small");
  mlstm::BwWorkspace bws = mlstm::carve_bw_workspace(bw_workspace, B, NH, S, DHQK, DHHV, stride, tiles);
  if (bw_workspace_bytes < bws.bytes) return fail("mlstm_hip_chunkwise_bw: backward workspace too small");
  hipStream_t st = (hipStream_t)stream;
  const int NC = (S + 127) / 128, BH = B * NH;
  const int sig = gate == MLSTM_GATE_SIG;
  const int use_nrow = !(sig && !normalize);
  const float qk_scale = 1.0f / sqrtf((float)DHQK);

  if (use_fused(path, DHQK, DHHV)) {
    if (f16) return fail("mlstm_hip_chunkwise_bw: the fused kernel path multiplies bf16 operands only");
    mlstm::FusedHvArgs fa;
    memset(&fa, 0, sizeof(fa));
    fa.Q = (const uint16_t*)q; fa.K = (const uint16_t*)k; fa.V = (const uint16_t*)v; fa.dH = (const uint16_t*)dH;
    fa.g = ws.g;
    fa.init = dC_last;
    fa.nrow = ws.nrow;
    fa.states = bws.dcstates;
    fa.Out = (uint16_t*)dV;
    fa.final_out = dC0;
    fa.S = S; fa.NC = NC; fa.DHQK = DHQK; fa.DHHV = DHHV;
    fa.qk_scale = qk_scale; fa.eps = eps;
    fa.sig_gate = sig; fa.use_nrow = use_nrow;
    fa.stride = stride;
    {
      ProfileScope ps("fused_dv", st);
      if (const char* e = mlstm::launch_fused_hv(fa, BH, /*is_dv=*/true, st)) return fail(e);
    }
    if (check_launch("fused_hv dV")) return 1;
  } else {
    mlstm::ScanArgs sa;
    memset(&sa, 0, sizeof(sa));
    sa.X = (const uint16_t*)q;
    sa.Y = (const uint16_t*)dH;
    sa.scale_a = ws.g.bbar;
    sa.nrow = use_nrow ? ws.nrow : nullptr;
    sa.gbar = ws.g.gbar;
    sa.init = dC_last;
    sa.states = bws.dcstates;
    sa.final_out = dC0;
    sa.S = S; sa.NC = NC; sa.DHQK = DHQK; sa.DHHV = DHHV;
    sa.qk_scale = qk_scale; sa.eps = eps;
    sa.backward = 1;
    sa.stride = stride;
    sa.f16 = f16;
    {
      ProfileScope ps("scan_bw", st);
      if (const char* e = mlstm::launch_scan(sa, BH, /*hilo=*/false, st)) return fail(e);
    }
    if (check_launch("scan_bw")) return 1;

    mlstm::ParHvArgs pv;
    memset(&pv, 0, sizeof(pv));
    pv.Q = (const uint16_t*)q; pv.K = (const uint16_t*)k; pv.V = (const uint16_t*)v; pv.dH = (const uint16_t*)dH;
    pv.g = ws.g;
    pv.states = bws.dcstates;
    pv.nrow = ws.nrow;
    pv.Out = (uint16_t*)dV;
    pv.S = S; pv.NC = NC; pv.DHQK = DHQK; pv.DHHV = DHHV;
    pv.qk_scale = qk_scale; pv.eps = eps;
    pv.sig_gate = sig; pv.use_nrow = use_nrow;
    pv.stride = stride;
    pv.f16 = f16;
    {
      ProfileScope ps("par_dv", st);
      if (const char* e = launch_hv(path, pv, BH, /*is_dv=*/true, st)) return fail(e);
    }
    if (check_launch("par_hv dV")) return 1;
  }

  mlstm::ParQkArgs pq;
  memset(&pq, 0, sizeof(pq));
  pq.Q = (const uint16_t*)q; pq.K = (const uint16_t*)k; pq.V = (const uint16_t*)v; pq.dH = (const uint16_t*)dH;
  pq.g = ws.g;
  pq.nrow = ws.nrow;
  pq.S = S; pq.NC = NC; pq.DHQK = DHQK; pq.DHHV = DHHV;
  pq.qk_scale = qk_scale; pq.eps = eps;
  pq.use_nrow = use_nrow;
  pq.stride = stride;
  pq.f16 = f16;
  // dQ and dK in one launch: the workgroups of a chunk run side by side and share the Q, K, V and dH rows they stream
  pq.states = ws.cstates; pq.Out = (uint16_t*)dQ; pq.rowdot = bws.qdq;
  pq.states2 = bws.dcstates; pq.Out2 = (uint16_t*)dK; pq.rowdot2 = bws.kdk;
  {
    ProfileScope ps("par_dqdk", st);
    if (const char* e = launch_qk(path, pq, BH, st)) return fail(e);
  }
  if (check_launch("par_qk dQ+dK")) return 1;

  mlstm::GateGradArgs ga;
  memset(&ga, 0, sizeof(ga));
  ga.i = i; ga.f = f; ga.qdq = bws.qdq; ga.kdk = bws.kdk; ga.dI = dI; ga.dF = dF;
  ga.ntiles = tiles;
  ga.S = S; ga.NC = NC; ga.dtype_gates = dtype_gates; ga.sig_gate = sig;
  {
    ProfileScope ps("gate_grads", st);
    if (const char* e = mlstm::launch_gate_grads(ga, BH, st)) return fail(e);
  }
  return check_launch("gate_grads");
}

}  // extern "C"
