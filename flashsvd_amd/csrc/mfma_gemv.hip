// Decode projections for 3..64 rows at once (batched decoding, token-tiled MLP) on the matrix cores.
//
// At batch 1 a projection is a row-dot GEMV on the vector ALU; from a handful of rows on, the vector
// path has to re-read the activations from LDS once per weight row and row of the batch and runs out of
// LDS bandwidth long before HBM is busy.  Here a wave owns 16 weight rows and a slice of K (2, 4 or 8 waves
// share one 16-row tile),
// each wave feeds 16 rows x 32 k of W (A operand) and 16 batch rows x 32 k of X (B operand, read straight
// from L2: the batch is tiny) to V_MFMA_F32_16X16X32_BF16 and accumulates a 16 x 16 fp32 tile per 16
// batch rows; the waves' tiles are added in wave order through LDS (deterministic) and the epilogue
// applies the rounding points of the vector kernels: bias, one bf16 rounding, residual, or SwiGLU.
#include "common.hpp"
#include "kernels.hpp"

namespace fsvd {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(1))) u32x4_t* gp16_t;

constexpr int kMfThreads = 512;
constexpr int kMfWaves = kMfThreads / 64;

__device__ __forceinline__ bf16x8_t ldw_frag(const uint16_t* p) {
  return __builtin_bit_cast(bf16x8_t, __builtin_nontemporal_load((gp16_t)(uintptr_t)p));
}
__device__ __forceinline__ bf16x8_t ldx_frag(const uint16_t* p) {
  return __builtin_bit_cast(bf16x8_t, *(gp16_t)(uintptr_t)p);
}


// NB: 16-row batch tiles (B <= 16 * NB); KS: waves that split K for one 16-row weight tile, so a workgroup
// of 8 waves covers 8 / KS weight tiles
template <int NB, bool DUAL, int KS>
__global__ __launch_bounds__(kMfThreads) void mfma_linear_kernel(MfmaArgs a) {
  constexpr int NM = DUAL ? 2 : 1;
  constexpr int RT = kMfWaves / KS;
  __shared__ float red[kMfWaves][NM][NB][4][64];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lr = lane & 15, lg = lane >> 4;
  const int rt = wave / KS, ks = wave % KS;
  const int n0 = (blockIdx.x * RT + rt) * 16;
  const int ksteps = a.K >> 5;
  // the KS waves of a weight tile take the k-steps in turn (wave ks: steps ks, ks + KS, ...), so that together they read
  // KS * 64 contiguous bytes of every row at a time; s counts this wave's own steps
  const int s0 = 0, s1 = (ksteps - ks + KS - 1) / KS;
  const int64_t wo = (int64_t)min(n0 + lr, a.N - 1) * a.ldw + lg * 8;
  const uint16_t* w0 = a.W + wo;
  const uint16_t* w1 = DUAL ? a.W2 + wo : nullptr;
  const uint16_t* xr[NB];
#pragma unroll
  for (int t = 0; t < NB; ++t) xr[t] = a.x + (int64_t)min(t * 16 + lr, a.B - 1) * a.ldx + lg * 8;
  f32x4_t acc[NM][NB];
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int t = 0; t < NB; ++t) acc[m][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  // four k-steps per trip, all loads of a trip requested before the first product; steps past the end of
  // this wave's slice read the last step again and contribute zero
  constexpr int UN = 4;
  const bf16x8_t zero = __builtin_bit_cast(bf16x8_t, u32x4_t{0u, 0u, 0u, 0u});
  for (int s = s0; s < s1; s += UN) {
    bf16x8_t fa0[UN], fa1[UN], fb0[UN][NB], fb1[UN][NB];
#pragma unroll
    for (int j = 0; j < UN; ++j) {
      const int k = (min(s + j, s1 - 1) * KS + ks) << 5;
      fa0[j] = ldw_frag(w0 + k);
      if (DUAL) fa1[j] = ldw_frag(w1 + k);
#pragma unroll
      for (int t = 0; t < NB; ++t) {
        fb0[j][t] = ldx_frag(xr[t] + k);
        if (DUAL) fb1[j][t] = ldx_frag(xr[t] + a.up_off + k);
      }
    }
#pragma unroll
    for (int j = 0; j < UN; ++j) {
      const bool live = s + j < s1;
      const bf16x8_t a0 = live ? fa0[j] : zero;
#pragma unroll
      for (int t = 0; t < NB; ++t) {
        acc[0][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, fb0[j][t], acc[0][t], 0, 0, 0);
        if (DUAL) acc[1][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(live ? fa1[j] : zero, fb1[j][t], acc[1][t], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int t = 0; t < NB; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][m][t][i][lane] = acc[m][t][i];
  __syncthreads();
  // one thread per output element of the RT tiles of 16 x (16 * NB): element i of lane l is row
  // (l / 16) * 4 + i, batch column l % 16; the KS partial tiles are added in wave order
  for (int o = tid; o < RT * NB * 256; o += kMfThreads) {
    const int q = o / (NB * 256), oo = o - q * (NB * 256);
    const int t = oo >> 8, r = oo & 255, i = r >> 6, l = r & 63;
    const int n = (blockIdx.x * RT + q) * 16 + (l >> 4) * 4 + i, b = t * 16 + (l & 15);
    float v0 = 0.f, v1 = 0.f;
#pragma unroll
    for (int w = 0; w < KS; ++w) {
      v0 += red[q * KS + w][0][t][i][l];
      if (DUAL) v1 += red[q * KS + w][NM - 1][t][i][l];
    }
    if (n >= a.N || b >= a.B) continue;
    float v;
    if (DUAL) {
      if (a.mode == 0) {
        v0 = round_bf16(v0);
        v1 = round_bf16(v1);
        v = round_bf16(round_bf16(silu_f32(v0)) * v1);
      } else {
        v = round_bf16((v0 * (1.0f / (1.0f + expf(-v0)))) * v1);
      }
    } else {
      if (a.bias) v0 += bf16_bits_to_f32(a.bias[n]);
      v = round_bf16(v0);
      if (a.res) v = round_bf16(bf16_bits_to_f32(a.res[(int64_t)b * a.ldres + n]) + v);
    }
    a.y[(int64_t)b * a.ldy + n] = (uint16_t)f32_to_bf16_bits(v);
  }
}

template <int NB, bool DUAL>
static void launch_mfma_ks(const MfmaArgs& a, int ks, hipStream_t st) {
  const int tiles = (a.N + 15) / 16;
  const dim3 block(kMfThreads);
  if (ks == 2) hipLaunchKernelGGL((mfma_linear_kernel<NB, DUAL, 2>), dim3((tiles + 3) / 4), block, 0, st, a);
  else if (ks == 4) hipLaunchKernelGGL((mfma_linear_kernel<NB, DUAL, 4>), dim3((tiles + 1) / 2), block, 0, st, a);
  else hipLaunchKernelGGL((mfma_linear_kernel<NB, DUAL, 8>), dim3(tiles), block, 0, st, a);
}

template <bool DUAL>
static int launch_mfma(const MfmaArgs& a0, hipStream_t st, const char* who) {
  // K is split over as few waves as still give every compute unit a workgroup: long slices amortise the
  // reduction, but a small matrix needs all eight waves of a workgroup on one weight tile to fill the chip
  const int tiles = (a0.N + 15) / 16, ksteps = a0.K >> 5;
  int ks = 8;
  for (int c = 2; c <= 8; c *= 2)
    if ((tiles * c + 7) / 8 >= 256 && ksteps / c >= 4) { ks = c; break; }
  // many rows (prefill): the tiled kernel reads every weight once per 128 rows instead of once per 64
  if (gemm_tiles_apply(a0)) return launch_gemm_tiles(a0, DUAL, st, who);
  // a batch of rows: 32-row tiles with K split over workgroups, when the caller has registered a workspace
  if (gemm_rows_apply(a0)) return launch_gemm_rows(a0, DUAL, st, who);
  // batches above 64 rows go in slices of 64
  for (int b0 = 0; b0 < a0.B; b0 += 64) {
    MfmaArgs a = a0;
    a.B = min(64, a0.B - b0);
    a.x = a0.x + (int64_t)b0 * a0.ldx;
    a.y = a0.y + (int64_t)b0 * a0.ldy;
    if (a0.res) a.res = a0.res + (int64_t)b0 * a0.ldres;
    const int nb = (a.B + 15) / 16;
    if (nb == 1) launch_mfma_ks<1, DUAL>(a, ks, st);
    else if (nb == 2) launch_mfma_ks<2, DUAL>(a, ks, st);
    else if (nb == 3) launch_mfma_ks<3, DUAL>(a, ks, st);
    else launch_mfma_ks<4, DUAL>(a, ks, st);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_last_error("%s: launch failed: %s", who, hipGetErrorString(e)); return kErrLaunch; }
  }
  return kOk;
}

static inline bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// true when the matrix-core path applies (the caller then skips the vector kernel)
bool mfma_linear_applies(const LinearArgs& a) {
  return a.B >= 3 && a.norm_w == nullptr && (a.K % 32) == 0 && (a.ldw % 8) == 0 && (a.ldx % 8) == 0 && al16(a.W) && al16(a.x);
}
int launch_linear_mfma(const LinearArgs& a, hipStream_t st) {
  MfmaArgs m{a.x, a.ldx, 0, a.W, nullptr, a.ldw, a.bias, a.res, a.ldres, a.y, a.ldy, a.B, a.N, a.K, 0};
  return launch_mfma<false>(m, st, "fsvd_linear");
}
bool mfma_swiglu_applies(const SwigluArgs& a) {
  return a.B >= 3 && (a.R % 32) == 0 && (a.ldw % 8) == 0 && (a.ldp % 8) == 0 && (a.up_off % 8) == 0 && al16(a.gate_u) &&
         al16(a.up_u) && al16(a.p);
}
int launch_swiglu_mfma(const SwigluArgs& a, hipStream_t st) {
  MfmaArgs m{a.p, a.ldp, a.up_off, a.gate_u, a.up_u, a.ldw, nullptr, nullptr, 0, a.h, a.ldh, a.B, a.D, a.R, a.mode};
  return launch_mfma<true>(m, st, "fsvd_swiglu_linear");
}

}  // namespace fsvd
