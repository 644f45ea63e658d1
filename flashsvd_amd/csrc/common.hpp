// Shared device helpers for the gfx950 kernels: bf16 packing, wave64 reductions,
// status codes of the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fsvd {

constexpr int kWave = 64;

// status codes returned by every extern "C" entry point (0 == ok)
enum Status : int {
  kOk = 0,
  kErrBadShape = -1,     // a dimension is out of the supported range
  kErrBadAlign = -2,     // pointer / stride alignment the kernel needs is missing
  kErrBadDtype = -3,
  kErrNullPtr = -4,
  kErrLaunch = -5,       // hipGetLastError() after the launch
  kErrWorkspace = -6,    // caller workspace too small
};

void set_last_error(const char* fmt, ...);

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }
__device__ __forceinline__ float bf16_lo(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t packed) { return __uint_as_float(packed & 0xffff0000u); }

// round-to-nearest-even fp32 -> bf16 (bit pattern in the low 16 bits)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  __bf16 h = static_cast<__bf16>(f);
  return static_cast<uint32_t>(__builtin_bit_cast(unsigned short, h));
}
// value after one bf16 rounding
__device__ __forceinline__ float round_bf16(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
}

// acc += a.lo*b.lo + a.hi*b.hi with fp32 accumulation (V_DOT2_F32_BF16)
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float acc) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), acc, false);
}
__device__ __forceinline__ float dot8_bf16(const u32x4_t& w, const u32x4_t& x, float acc) {
  acc = dot2_bf16(w.x, x.x, acc);
  acc = dot2_bf16(w.y, x.y, acc);
  acc = dot2_bf16(w.z, x.z, acc);
  acc = dot2_bf16(w.w, x.w, acc);
  return acc;
}

// The 16-bit element types of the fused product kernels (dtype codes of the C ABI: 0 = bf16, 1 = fp16).  The kernels
// move bit patterns; an element type says how a pattern widens to fp32, how fp32 rounds to it (nearest even, as
// torch does) and which packed dot-product instruction multiplies it (fp32 accumulation in both).
// frag_t / mfma: eight elements as a matrix-core operand and V_MFMA_F32_16X16X32_{BF16,F16}.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
template <int DT> struct E16;
template <> struct E16<0> {
  static constexpr int code = 0;
  // int4 streams: nib<S>(d) turns the nibbles at bits S and S + 16 of d into the patterns of two elements nib_off + n
  // (exact in the element type) without a conversion: here 0x4300 | n = 128 + n.  one2 is the pair (1, 1).
  static constexpr uint32_t one2 = 0x3f803f80u;
  static constexpr int nib_off = 128;
  template <int S> static __device__ __forceinline__ uint32_t nib(uint32_t d) { return ((d >> S) & 0x000f000fu) | 0x43004300u; }
  typedef bf16x8_t frag_t;
  static __device__ __forceinline__ f32x4_t mfma(frag_t a, frag_t b, f32x4_t c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ float lo(uint32_t packed) { return bf16_lo(packed); }
  static __device__ __forceinline__ float hi(uint32_t packed) { return bf16_hi(packed); }
  static __device__ __forceinline__ float val(uint32_t h) { return bf16_bits_to_f32(h); }      // pattern in the low 16 bits
  static __device__ __forceinline__ uint32_t bits(float f) { return f32_to_bf16_bits(f); }
  static __device__ __forceinline__ float rnd(float f) { return round_bf16(f); }
  static __device__ __forceinline__ uint32_t pack2(float l, float h) { return pack_bf16x2(l, h); }
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) { return dot2_bf16(a, b, acc); }
  static __device__ __forceinline__ float dot8(const u32x4_t& w, const u32x4_t& x, float acc) { return dot8_bf16(w, x, acc); }
};
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
template <> struct E16<1> {
  static constexpr int code = 1;
  // 0x4c00 | n << 6 = 16 + n: the nibble sits in the top of the mantissa, so the offset that the products carry (and
  // that the row sum takes out again) stays small against the weights themselves
  static constexpr uint32_t one2 = 0x3c003c00u;
  static constexpr int nib_off = 16;
  template <int S> static __device__ __forceinline__ uint32_t nib(uint32_t d) {
    return ((S < 6 ? d << (S < 6 ? 6 - S : 0) : d >> (S < 6 ? 0 : S - 6)) & 0x03c003c0u) | 0x4c004c00u;
  }
  typedef f16x8_t frag_t;
  static __device__ __forceinline__ f32x4_t mfma(frag_t a, frag_t b, f32x4_t c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
  // V_CVT_F32_F16 on the low half of a 32-bit register, written as an instruction: left to the compiler, the widening is
  // folded into mixed-precision multiply-adds on 16-bit subregisters, which makes it copy whole register arrays whenever
  // one element of them is rewritten (the step kernel's staging went from 150 registers to 256 with 780 spills)
  static __device__ __forceinline__ float val(uint32_t h) {
    float f;
    asm("v_cvt_f32_f16 %0, %1" : "=v"(f) : "v"(h));
    return f;
  }
  static __device__ __forceinline__ float lo(uint32_t packed) { return val(packed); }               // the instruction reads the low half
  static __device__ __forceinline__ float hi(uint32_t packed) { return val(packed >> 16); }
  static __device__ __forceinline__ uint32_t bits(float f) {
    return static_cast<uint32_t>(__builtin_bit_cast(unsigned short, static_cast<_Float16>(f)));
  }
  static __device__ __forceinline__ float rnd(float f) { return (float)static_cast<_Float16>(f); }
  static __device__ __forceinline__ uint32_t pack2(float l, float h) { return bits(l) | (bits(h) << 16); }
  // V_DOT2_F32_F16
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, a), __builtin_bit_cast(f16x2_t, b), acc, false);
  }
  static __device__ __forceinline__ float dot8(const u32x4_t& w, const u32x4_t& x, float acc) {
    acc = dot2(w.x, x.x, acc);
    acc = dot2(w.y, x.y, acc);
    acc = dot2(w.z, x.z, acc);
    acc = dot2(w.w, x.w, acc);
    return acc;
  }
};

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
// sum over each aligned group of 16 lanes; every lane of the group gets the sum
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_f32<0x141>(v);  // row_half_mirror
  v += dpp_f32<0x140>(v);  // row_mirror
  return v;
}
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, dpp_f32<0xB1>(v));
  v = fmaxf(v, dpp_f32<0x4E>(v));
  v = fmaxf(v, dpp_f32<0x141>(v));
  v = fmaxf(v, dpp_f32<0x140>(v));
  return v;
}
// sum over the 64 lanes of the wave; the result is wave-uniform
__device__ __forceinline__ float wave_sum(float v) {
  v = row16_sum(v);
  float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
  float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return (a + b) + (c + d);
}
__device__ __forceinline__ float wave_max(float v) {
  v = row16_max(v);
  float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
  float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return fmaxf(fmaxf(a, b), fmaxf(c, d));
}

// Cross-workgroup hand-off without L2 write-back/invalidate fences: producers use write-through
// (agent-scope) stores, wait until the memory system has acknowledged them, then signal through an
// agent-scope atomic; consumers read with agent-scope loads.  A workgroup-scope release fence does
// not wait for outstanding stores on this target, hence the explicit wait.
__device__ __forceinline__ void wait_stores_acked() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_waitcnt(0);   // vmcnt(0) expcnt(0) lgkmcnt(0)
}

// Workgroups are handed to the eight XCDs in turn (linear id % 8) and every XCD has an L2 of its own.  Position of
// workgroup `linear` of `total` in an order that gives each XCD one contiguous run: workgroups that read the same
// operands sit next to each other in that order and so share an L2.
__device__ __forceinline__ int xcd_run_index(int linear, int total) {
  const int xcd = linear & 7, q = total >> 3, rem = total & 7;
  return xcd * q + min(xcd, rem) + (linear >> 3);
}

__device__ __forceinline__ float silu_f32(float x) { return x / (1.0f + expf(-x)); }

}  // namespace fsvd
