/*
 * mlstm_hip.h -- C ABI of libmlstm_hip.so: the mLSTM hot path (TFLA chunkwise forward/backward and the
 * fused recurrent decode step) as hand-written gfx950 HIP kernels.
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer owned by the caller; the library never allocates or frees device
 *     memory and keeps no state between calls except a thread-local error string (and, while the optional
 *     per-kernel timing is enabled, host-side event records).
 *   - Tensors are dense row-major: q,k (B,NH,S,DHQK); v,H,dH (B,NH,S,DHHV); i,f (B,NH,S);
 *     C (B,NH,DHQK,DHHV) fp32; n (B,NH,DHQK) fp32; m (B,NH) fp32.
 *   - `stream` is a hipStream_t passed as void*; launches are asynchronous on it.
 *   - Return value 0 = success; anything else = failure, message via mlstm_hip_last_error().
 *   - dtype codes: MLSTM_F32 = 0, MLSTM_BF16 = 1, MLSTM_F16 = 2.  The chunkwise entry points take q/k/v (and dH) in
 *     bf16 or fp16 and multiply in that format on the matrix cores with fp32 accumulation (the kept chunk states are
 *     rounded to the same format; fp16 has three more mantissa bits and overflows above 65504); gates in fp32, bf16 or
 *     fp16.  MLSTM_F32 is rejected for the q/k/v of a chunkwise call: there is no fp32 matrix path.  (The Python host
 *     code converts float32 tensors to bf16 before the call, so a float32 call there computes with bf16 operands --
 *     about 1e-2 relative error of the outputs in norm -- and not in the fp32 arithmetic of the reference's float32
 *     configuration.)  The decode entry points take q/k/v, gates and states in fp32, bf16 or fp16 each (fp32 arithmetic).
 *   - gate codes: MLSTM_GATE_EXP = 0 (mLSTMexp), MLSTM_GATE_SIG = 1 (mLSTMsig, sigmoid input gate).
 *   - Supported shapes: DHQK % 64 == 0 (at most 896), DHHV % 64 == 0, any S >= 1 (the kernels mask the ragged tail).
 *
 * Each entry point names the reference interface it replaces (paths relative to the reference checkout).
 */
#ifndef MLSTM_HIP_H
#define MLSTM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MLSTM_F32 0
#define MLSTM_BF16 1
#define MLSTM_F16 2
#define MLSTM_GATE_EXP 0
#define MLSTM_GATE_SIG 1

/* ABI version of the loaded library (bumped on any signature change). */
int mlstm_hip_abi_version(void);

/*
 * Per-kernel timing for benchmarks (no counterpart in the reference, which times whole operator calls with
 * torch events: mlstm_kernels/utils/benchmark/runtime.py:30-170).  While enabled, every kernel launch of this
 * library is bracketed by HIP events on its launch stream.  mlstm_hip_profile_read(0, ...) waits for the
 * recorded events, aggregates them by kernel name and returns the number of distinct kernels; entry `index`
 * (name, summed milliseconds, number of launches) is copied out.  Host-side bookkeeping only.
 */
int mlstm_hip_profile_enable(int on);
int mlstm_hip_profile_read(int index, char* name, size_t name_cap, float* total_ms, int* launches);

/* Message of the last failure on the calling thread ("" if none). */
const char* mlstm_hip_last_error(void);

/*
 * Per-call tuning options of the chunkwise entry points (no state is kept between calls).
 *
 * path: kernel selection for the value-column side of the passes (H forward, dV backward).  No counterpart in the
 * reference, whose Triton kernels are always the two-kernel form, recurrent_fw_C followed by parallel_fw_Hintra
 * (mlstm_kernels/torch/chunkwise/triton_xl_chunk/fw.py:20-136).
 *   MLSTM_PATH_AUTO  : the fastest one for the shape as measured on MI355X: the streaming H / dV kernels where the
 *                      conditions of MLSTM_PATH_STREAM hold, the window dQ / dK kernel (windows of two chunks that
 *                      share a kept state) at state_stride 2 with DHQK = 256, DHHV a multiple of 64 and S a multiple
 *                      of 256, the kernels of MLSTM_PATH_SPLIT for everything else
 *   MLSTM_PATH_SPLIT : state scan + chunk-parallel kernel over materialised chunk states
 *   MLSTM_PATH_STREAM: the split form with the chunk-parallel kernels as persistent workgroups whose waves are split
 *                      into producers (global memory -> LDS, several slabs in flight) and consumers (matrix
 *                      instructions); DHQK = 256, DHHV a multiple of 512 (exactly 512 with a head norm), S a
 *                      multiple of 128: other shapes are rejected.  dQ / dK: the window kernel under the conditions above, else a
 *                      streaming kernel per chunk and gradient.  Same workspaces as MLSTM_PATH_SPLIT.
 *   MLSTM_PATH_FUSED : one sequential kernel per pass, state slice resident in registers (DHQK = 128 or 256 only:
 *                      other head dimensions are rejected)
 *
 * state_stride: a chunk state (DHQK x DHHV bf16 per chunk of 128 positions and head) is kept every state_stride
 * chunks; chunks in between reach back to the nearest kept state through additional score blocks.  Replaces the
 * reference's chunk_size_inter / chunk_size_intra pair with save_states_every_nth_chunk =
 * chunk_size_intra / chunk_size_inter (mlstm_kernels/triton/chunkwise/kernel_param_heuristics.py:28-31,118-121):
 * chunk_size_inter is fixed at 128 here and state_stride = chunk_size_intra / 128.  0 = the default for the shape,
 * otherwise 1 .. 8.  Results agree for every value within the rounding of bf16 operands.
 *
 * The forward (with keep_for_backward), both workspace queries and the backward of one pass must be called with the
 * same path and state_stride: they decide the layout of the workspaces.
 */
#define MLSTM_PATH_AUTO 0
#define MLSTM_PATH_SPLIT 1
#define MLSTM_PATH_FUSED 2
#define MLSTM_PATH_STREAM 3

/*
 * head_norm: optional normalisation of every row of H over its DHHV columns, fused into the epilogue of the forward
 * output kernel -- the op that follows the mLSTM cell in the xLSTM block and that the reference's backward convention
 * assumes (mlstm_kernels/torch/chunkwise/native/bw.py:44-46); the reference states the norm itself in
 * mlstm_kernels/utils/analysis/transfer_behavior/_norm_layers.py:11-35 (layer_normalize / rms_normalize: fp32
 * reductions over the last dimension, no scale parameters).  With MLSTM_NORM_LAYER or MLSTM_NORM_RMS the forward
 * writes the normalised rows into H (the un-normalised output never goes to memory) and the per-row mean (0 for rms)
 * and reciprocal standard deviation into norm_mean / norm_rstd (fp32 (B,NH,S)).  Needs DHHV = 64, 128, 256 or 512 and
 * the split kernel path.  mlstm_hip_head_norm_bw turns the gradient of the normalised rows into the gradient of H,
 * which mlstm_hip_chunkwise_bw takes as dH.
 */
#define MLSTM_NORM_NONE 0
#define MLSTM_NORM_LAYER 1
#define MLSTM_NORM_RMS 2

/*
 * Fused recurrent decode step (one token for every (b, head)).
 * Replaces: mlstm_kernels/torch/recurrent/triton_step.py:15-127 (mlstm_recurrent_step__triton_fw) and the
 * Triton kernel mlstm_kernels/triton/recurrent/fw_step_fused.py:19-195.
 *   q,k (B,NH,DHQK), v (B,NH,DHHV) in dtype_qkv; i,f (B,NH) in dtype_gates; h (B,NH,DHHV) in dtype_qkv.
 *   States C (B,NH,DHQK,DHHV), n (B,NH,DHQK), m (B,NH) in and out in dtype_state (MLSTM_F32, MLSTM_BF16 or MLSTM_F16: the
 *   reference's dtype_state, triton_step.py:33,67-69); the arithmetic is fp32 either way, h is formed from the
 *   unrounded new state.  DHHV % 4 == 0 (fp32 state) or % 8 == 0 (16-bit state).
 *   c_out may alias c_in (in-place update of the state matrix); n_out/m_out must be distinct from n_in/m_in
 *   (every workgroup of a head reads the old n and m while one of them writes the new values).
 */
int mlstm_hip_step(const void* q, const void* k, const void* v, const void* i, const void* f,
                   const void* c_in, const void* n_in, const void* m_in,
                   void* h, void* c_out, void* n_out, void* m_out,
                   int B, int NH, int DHQK, int DHHV, float eps,
                   int dtype_qkv, int dtype_gates, int dtype_state, void* stream);

/*
 * Recurrent mLSTM over T tokens in one launch (multi-token decode, the remainder of a prefill): the step above
 * applied T times with the state held on chip -- C is read once before the first token and written once after the
 * last, instead of once each way per token.
 * Replaces: the token loop mlstm_kernels/torch/recurrent/native_sequence.py:13-122
 * (mlstm_recurrent_sequence__triton_step_fused_fw = _mlstm_recurrent_sequence_loop_fw over the fused step).
 *   q,k (B,NH,T,DHQK), v (B,NH,T,DHHV) in dtype_qkv; i,f (B,NH,T) in dtype_gates; h (B,NH,T,DHHV) in dtype_qkv;
 *   states as for mlstm_hip_step (dtype_state; between tokens the state stays fp32 in registers, so a bf16 state is
 *   rounded once per call, not once per token; c_out may alias c_in, n_out/m_out must be distinct from n_in/m_in).
 *   DHQK <= 1024.
 */
int mlstm_hip_recurrent_sequence(const void* q, const void* k, const void* v, const void* i, const void* f,
                                 const void* c_in, const void* n_in, const void* m_in,
                                 void* h, void* c_out, void* n_out, void* m_out,
                                 int B, int NH, int T, int DHQK, int DHHV, float eps,
                                 int dtype_qkv, int dtype_gates, int dtype_state, void* stream);

/*
 * Bytes of caller-provided workspace the chunkwise forward needs.  With keep_for_backward != 0 the
 * workspace additionally holds everything the backward re-uses (gate vectors, per-chunk bf16 states,
 * per-row normalisers) and must be handed unchanged to mlstm_hip_chunkwise_bw.
 */
size_t mlstm_hip_chunkwise_fw_workspace_bytes(int B, int NH, int S, int DHQK, int DHHV, int keep_for_backward,
                                              int path, int state_stride);

/*
 * TFLA chunkwise forward, mLSTMexp or mLSTMsig.
 * Replaces: mlstm_kernels/torch/chunkwise/triton_xl_chunk/fw.py:20-136 (mlstm_chunkwise_fw: recurrent_fw_C +
 * parallel_fw_Hintra + gate pre-pass) and .../triton_xl_chunk_siging/fw.py for gate == MLSTM_GATE_SIG.
 *   c0,n0,m0: initial states or NULL (all three NULL together; m0 ignored for the sig gate).
 *   H (B,NH,S,DHHV) in dtype_qkv.  n_out, m_out: optional fp32 (B,NH,S) per-row normaliser max(|den|,floor)
 *   and stabiliser (NULL to skip).  c_last,n_last,m_last: optional fp32 last states (NULL to skip).
 *   With c_last given, the state scan carries the gated values as a 16-bit head plus a 16-bit remainder in every
 *   chunk that still weighs at least 2^-8 in the last state, so c_last is accurate to ~1e-5 relative; with c_last
 *   NULL it rounds them once (as the replaced kernels do), which is up to a fifth faster and changes H only within
 *   the tolerance of its 16-bit operands.
 *   MLSTM_PATH_FUSED takes bf16 only.
 *   normalize applies to the sig gate only (0: H is the bare numerator).
 */
int mlstm_hip_chunkwise_fw(const void* q, const void* k, const void* v, const void* i, const void* f,
                           const float* c0, const float* n0, const float* m0,
                           void* H, float* n_out, float* m_out,
                           float* c_last, float* n_last, float* m_last,
                           void* workspace, size_t workspace_bytes, int keep_for_backward,
                           int B, int NH, int S, int DHQK, int DHHV, float eps,
                           int dtype_qkv, int dtype_gates, int gate, int normalize, int path, int state_stride,
                           int head_norm, float norm_eps, float* norm_mean, float* norm_rstd, void* stream);

/*
 * Saved-state policy of the reference (recompute_states_in_bw, mlstm_kernels/torch/chunkwise/triton_xl_chunk/fwbw.py:45-62
 * and bw.py:75-95: the forward keeps no chunk states and the backward runs the state recurrence again).  The chunk
 * states are the last and by far the largest part of the forward workspace; a caller that wants to hold less memory
 * between forward and backward keeps only the first mlstm_hip_chunkwise_fw_saved_bytes() bytes of it (gate vectors,
 * normaliser states, row normalisers: independent of state_stride), and before the backward copies them to the start
 * of a full-size workspace and calls mlstm_hip_chunkwise_recompute_states, which runs the forward state scan again
 * and writes the chunk states behind them (k, v, c0, dtype_qkv, state_stride as in the forward call; c0 NULL = zero
 * initial state).  The workspace is then what mlstm_hip_chunkwise_bw expects.  The recomputed states equal the
 * forward's bit for bit when the forward returned no last state (c_last NULL); a forward that returned it carried a
 * remainder of the value operand in its late chunks, and the recomputed states of those chunks differ from the
 * forward's by one 16-bit rounding of that operand.
 */
size_t mlstm_hip_chunkwise_fw_saved_bytes(int B, int NH, int S, int DHQK, int DHHV);
int mlstm_hip_chunkwise_recompute_states(const void* k, const void* v, const float* c0,
                                         void* workspace, size_t workspace_bytes,
                                         int B, int NH, int S, int DHQK, int DHHV,
                                         int dtype_qkv, int state_stride, void* stream);

/*
 * Backward of the fused head norm: dX = rstd * (dY - mean_D(dY) - Y * mean_D(dY * Y)) for MLSTM_NORM_LAYER,
 * dX = rstd * (dY - Y * mean_D(dY * Y)) for MLSTM_NORM_RMS, per row of D = 64, 128, 256 or 512 values.
 * Replaces the autograd backward of the reference's layer_normalize / rms_normalize
 * (mlstm_kernels/utils/analysis/transfer_behavior/_norm_layers.py:11-35).  dY, Y, dX: (rows, D) in dtype (bf16 or fp16);
 * rstd: (rows) fp32 as written by the forward.
 */
int mlstm_hip_head_norm_bw(const void* dY, const void* Y, const float* rstd, void* dX, size_t rows, int D,
                           int head_norm, int dtype, void* stream);

/*
 * Allocation-free chunkwise forward (inference / prefill: nothing is kept for a backward pass).
 * No counterpart in the reference.  For callers that cannot allocate device memory around the call -- code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc: same arguments and results as
 * mlstm_hip_chunkwise_fw with keep_for_backward = 0, path = MLSTM_PATH_AUTO, state_stride = 0 and no head norm, but the workspace is
 * a static device array of MLSTM_NOALLOC_SCRATCH_BYTES inside the library (one copy per GPU, held until the process
 * ends) instead of a caller-provided buffer.  The call allocates and frees nothing.  Shapes whose workspace
 * (mlstm_hip_chunkwise_fw_workspace_bytes(B, NH, S, DHQK, DHHV, 0, MLSTM_PATH_AUTO, 0)) exceeds the static scratch are
 * rejected.  All calls on one GPU share that GPU's scratch: calls that overlap in time on one GPU race.
 * Under HIP graph capture: make one eager call of the same shape on the device before the capture begins.  The first
 * call on a device looks up the scratch address (hipGetSymbolAddress), the number of CUs and the kernels' LDS limits
 * (hipFuncSetAttribute), none of which a capturing stream records; later calls only launch kernels.
 */
#define MLSTM_NOALLOC_SCRATCH_BYTES (64u << 20)
int mlstm_hip_chunkwise_fw_noalloc(const void* q, const void* k, const void* v, const void* i, const void* f,
                                   const float* c0, const float* n0, const float* m0,
                                   void* H, float* n_out, float* m_out,
                                   float* c_last, float* n_last, float* m_last,
                                   int B, int NH, int S, int DHQK, int DHHV, float eps,
                                   int dtype_qkv, int dtype_gates, int gate, int normalize, void* stream);

/* Bytes of scratch the chunkwise backward needs in addition to the forward workspace. */
size_t mlstm_hip_chunkwise_bw_workspace_bytes(int B, int NH, int S, int DHQK, int DHHV, int state_stride);

/*
 * TFLA chunkwise backward (normaliser and stabilisers are constants, as in the reference).
 * Replaces: mlstm_kernels/torch/chunkwise/triton_xl_chunk/bw.py:27-227 (mlstm_chunkwise_bw: recurrent_bw_dC,
 * parallel_bw_dV/dK/dQ, gate-gradient post-pass) and the siging counterpart.
 *   fw_workspace: the forward's workspace, produced with keep_for_backward != 0 for the same inputs.
 *   dH (B,NH,S,DHHV) in dtype_qkv; dC_last optional fp32 gradient of the last C state (NULL = zero).
 *   dQ,dK (B,NH,S,DHQK), dV (B,NH,S,DHHV) in dtype_qkv; dI,dF fp32 (B,NH,S);
 *   dC0 optional fp32 (B,NH,DHQK,DHHV) gradient of the initial C state (NULL to skip).
 */
int mlstm_hip_chunkwise_bw(const void* q, const void* k, const void* v, const void* i, const void* f,
                           const void* dH, const float* dC_last,
                           void* dQ, void* dK, void* dV, float* dI, float* dF, float* dC0,
                           const void* fw_workspace, size_t fw_workspace_bytes,
                           void* bw_workspace, size_t bw_workspace_bytes,
                           int B, int NH, int S, int DHQK, int DHHV, float eps,
                           int dtype_qkv, int dtype_gates, int gate, int normalize, int path, int state_stride,
                           void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MLSTM_HIP_H */
