// Shared device helpers for the gfx950 mLSTM kernels: vector types, bf16 packing, MFMA wrappers,
// LDS fragment reads (plain and transposing), wave-level scans.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mlstm {

constexpr int kWave = 64;
constexpr int kChunk = 128;  // internal chunk length L of every chunkwise kernel

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
// 16 raw bytes as a native vector: unlike HIP's uint4 struct, a memory-to-memory copy through an array of these
// is promoted to registers (struct copies become memcpy calls the optimiser leaves in scratch memory)
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
// 8 bf16 (or fp16) as raw bits; convertible to the MFMA operand type without data movement
union Frag {
  uint4 u;
  bf16x8 v;
  f16x8 hv;
  uint16_t h[8];
  uint32_t w[4];
  uint2 d[2];
};

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

// round-to-nearest-even fp32 -> bf16 bits (finite inputs; NaN stays NaN via the quiet bit)
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
// two fp32 -> packed bf16x2 (round to nearest even) with the gfx950 hardware conversion v_cvt_pk_bf16_f32
typedef __bf16 bf16x2_hw __attribute__((ext_vector_type(2)));
typedef float f32x2_hw __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2_hw v = {lo, hi};
  const bf16x2_hw b = __builtin_convertvector(v, bf16x2_hw);
  uint32_t u;
  __builtin_memcpy(&u, &b, 4);
  return u;
}

// D(32x32) += A(32x16) * B(16x32), bf16 operands, fp32 accumulate.
// lane l: r = l % 32, h = l / 32.  A frag: A[r][8h..8h+7]; B frag: B[8h..8h+7][r];
// acc[i] = D[8*(i/4) + 4h + (i%4)][r].
__device__ __forceinline__ void mfma32(f32x16& acc, const Frag& a, const Frag& b) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, acc, 0, 0, 0);
}


// The chunkwise kernels multiply either bfloat16 (F16 = false) or float16 (F16 = true) operands; the accumulators,
// gates, normalisers and row scales are fp32 either way.  Element helpers for both 16-bit formats:
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
template <bool F16>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {  // two fp32 -> one packed pair, round to nearest even
  if constexpr (F16) {
    const f16x2 hv = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, hv);
  } else {
    return pack_bf16x2(lo, hi);
  }
}
template <bool F16>
__device__ __forceinline__ float lo2(uint32_t w) {  // low element of a packed pair
  if constexpr (F16) return (float)__builtin_bit_cast(f16x2, w)[0];
  else return __uint_as_float(w << 16);
}
template <bool F16>
__device__ __forceinline__ float hi2(uint32_t w) {  // high element of a packed pair
  if constexpr (F16) return (float)__builtin_bit_cast(f16x2, w)[1];
  else return __uint_as_float(w & 0xffff0000u);
}
template <bool F16>
__device__ __forceinline__ float elem_to_f32(uint16_t b) {
  if constexpr (F16) return (float)__builtin_bit_cast(_Float16, b);
  else return bf16_bits_to_f32(b);
}
template <bool F16>
__device__ __forceinline__ uint16_t f32_to_elem(float x) {
  if constexpr (F16) return __builtin_bit_cast(uint16_t, (_Float16)x);
  else return f32_to_bf16_bits(x);
}
template <bool F16>
__device__ __forceinline__ void mfma32(f32x16& acc, const Frag& a, const Frag& b) {
  if constexpr (F16) acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a.hv, b.hv, acc, 0, 0, 0);
  else acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, acc, 0, 0, 0);
}

typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

// Transposing 64-bit LDS read.  Within each block of 16 lanes, lane i must pass the address of the 4
// consecutive 16-bit elements T[k0 + i/4][n0 + 4*(i%4) .. +3]; it receives T[k0 .. k0+3][n0 + i].
__device__ __forceinline__ uint2 lds_read_tr16(const void* p) {
  s16x4 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p));
  union { s16x4 s; uint2 u; } c;
  c.s = r;
  return c.u;
}

// A copy of x the optimiser knows nothing about.  Index arithmetic derived from it inside a loop body is redone in
// every iteration instead of being hoisted out of the loop into registers that stay live (and get spilled) for the
// whole kernel; the handful of integer instructions per iteration is far cheaper than a spill reload, which queues
// behind the global loads in flight.
__device__ __forceinline__ int opaque(int x) {
  asm volatile("" : "+v"(x));
  return x;
}

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o);
  return x;
}
__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o));
  return x;
}

__device__ __forceinline__ float log_sigmoid(float x) {
  // log(sigmoid(x)) = min(x, 0) - log1p(exp(-|x|))
  return fminf(x, 0.f) - log1pf(expf(-fabsf(x)));
}

// dtype: 0 float32, 1 bfloat16, 2 float16
__device__ __forceinline__ float load_scalar(const void* p, size_t idx, int dtype) {
  if (dtype == 0) return ((const float*)p)[idx];
  if (dtype == 1) return bf16_bits_to_f32(((const uint16_t*)p)[idx]);
  return (float)((const _Float16*)p)[idx];
}

// Recurrent states may be kept in float32 (0), bfloat16 (1) or float16 (2); the arithmetic is float32.
__device__ __forceinline__ float load_state_scalar(const void* p, size_t idx, int sdt) {
  if (sdt == 0) return ((const float*)p)[idx];
  if (sdt == 1) return bf16_bits_to_f32(((const uint16_t*)p)[idx]);
  return (float)((const _Float16*)p)[idx];
}
__device__ __forceinline__ void store_state_scalar(void* p, size_t idx, int sdt, float x) {
  if (sdt == 0) ((float*)p)[idx] = x;
  else if (sdt == 1) ((uint16_t*)p)[idx] = f32_to_bf16_bits(x);
  else ((_Float16*)p)[idx] = (_Float16)x;
}
// two 16-bit state values packed in one 32-bit word (sdt = 1 or 2)
__device__ __forceinline__ void unpack_state2(uint32_t w, int sdt, float& lo, float& hi) {
  if (sdt == 1) {
    lo = __uint_as_float(w << 16);
    hi = __uint_as_float(w & 0xffff0000u);
  } else {
    const f16x2 hv = __builtin_bit_cast(f16x2, w);
    lo = (float)hv[0];
    hi = (float)hv[1];
  }
}
__device__ __forceinline__ uint32_t pack_state2(float lo, float hi, int sdt) {
  if (sdt == 1) return pack_bf16x2(lo, hi);
  const f16x2 hv = {(_Float16)lo, (_Float16)hi};
  return __builtin_bit_cast(uint32_t, hv);
}

// XCD-aware workgroup renumbering.  The hardware deals consecutive linear workgroup ids round-robin to the 8
// XCDs (each with its own L2).  Mapping linear id -> (id % 8) * (total / 8) + id / 8 gives every XCD a
// contiguous range of virtual ids, so neighbouring tiles (which share operands) share an L2.
struct BlockId {
  int x, y, z;
};
__device__ __forceinline__ BlockId xcd_block_id() {
  BlockId b = {(int)blockIdx.x, (int)blockIdx.y, (int)blockIdx.z};
  const int gx = gridDim.x, gy = gridDim.y, total = gx * gy * (int)gridDim.z;
  if (total % 8 == 0) {
    const int lin = b.x + gx * (b.y + gy * b.z);
    const int virt = (lin % 8) * (total / 8) + lin / 8;
    b.x = virt % gx;
    b.y = (virt / gx) % gy;
    b.z = virt / (gx * gy);
  }
  return b;
}

// LDS write of one 16-byte global vector (8 consecutive head-dim entries) in the fragment order used for
// every contraction over DHQK: inside each group of 16, entry 8a + 4h + c is stored at 8h + 4a + c.
__device__ __forceinline__ void store_perm16(uint16_t* row, int cv, uint4 v) {
  const int s16 = (cv >> 1) * 16, a = cv & 1;
  *(uint2*)(row + s16 + 4 * a) = make_uint2(v.x, v.y);
  *(uint2*)(row + s16 + 8 + 4 * a) = make_uint2(v.z, v.w);
}
__device__ __forceinline__ int perm16(int d) {  // position of head-dim entry d in fragment order
  const int s16 = d & ~15, a = (d >> 3) & 1, hh = (d >> 2) & 1, c = d & 3;
  return s16 + 8 * hh + 4 * a + c;
}

}  // namespace mlstm
