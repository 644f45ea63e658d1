// Batch-1..4 decode projections on nn.Linear-layout weights W[N,K] (row = one output):
// every row is one contiguous bf16 stream, a wave (or a whole workgroup for long rows)
// walks it with 16-byte loads, the activation vector sits in LDS as packed bf16, products
// go through V_DOT2_F32_BF16 with fp32 accumulation and the 64 lanes are folded with DPP.
// Epilogues reproduce the rounding points of a chain of bf16 nn.Linear modules.
#include "common.hpp"
#include "kernels.hpp"

namespace fsvd {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;

// ---------------------------------------------------------------------------------------
// stage the activation rows of one batch tile into LDS (packed bf16), optionally RMS-normed
//   xs layout: [BATCH][Kp] bf16, Kp = K rounded up to 8
// ---------------------------------------------------------------------------------------
template <int DT, int BATCH>
__device__ __forceinline__ void stage_x(const uint16_t* __restrict__ x, int64_t ldx, int nb, int K, int Kp,
                                        const uint16_t* __restrict__ norm_w, float eps, uint16_t* xs, float* red) {
  typedef E16<DT> E;
  const int tid = threadIdx.x;
  const bool vec = ((K & 7) == 0) && ((ldx & 7) == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0);
  for (int b = 0; b < BATCH; ++b) {
    uint16_t* dst = xs + b * Kp;
    if (b >= nb) {
      for (int k = tid; k < Kp; k += kThreads) dst[k] = 0;
      continue;
    }
    const uint16_t* src = x + (int64_t)b * ldx;
    if (norm_w == nullptr) {
      if (vec) {
        for (int k = tid * 8; k < K; k += kThreads * 8)
          *reinterpret_cast<u32x4_t*>(dst + k) = *reinterpret_cast<const u32x4_t*>(src + k);
      } else {
        for (int k = tid; k < Kp; k += kThreads) dst[k] = k < K ? src[k] : (uint16_t)0;
      }
      continue;
    }
    // RMSNorm: y = w * bf16(x * rsqrt(mean(x^2) + eps)), sum in fp32
    const bool vnorm = vec && ((reinterpret_cast<uintptr_t>(norm_w) & 15) == 0);
    float ss = 0.f;
    if (vnorm) {
      for (int k = tid * 8; k < K; k += kThreads * 8) {
        const u32x4_t v = *reinterpret_cast<const u32x4_t*>(src + k);
        const float a0 = E::lo(v.x), a1 = E::hi(v.x), a2 = E::lo(v.y), a3 = E::hi(v.y);
        const float a4 = E::lo(v.z), a5 = E::hi(v.z), a6 = E::lo(v.w), a7 = E::hi(v.w);
        ss += ((a0 * a0 + a1 * a1) + (a2 * a2 + a3 * a3)) + ((a4 * a4 + a5 * a5) + (a6 * a6 + a7 * a7));
      }
    } else {
      for (int k = tid; k < K; k += kThreads) {
        float v = E::val(src[k]);
        ss += v * v;
      }
    }
    ss = wave_sum(ss);
    __syncthreads();  // red[] free
    if ((tid & 63) == 0) red[tid >> 6] = ss;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) tot += red[w];
    const float rs = rsqrtf(tot / (float)K + eps);
    if (vnorm) {
      for (int k = tid * 8; k < K; k += kThreads * 8) {
        const u32x4_t v = *reinterpret_cast<const u32x4_t*>(src + k);
        const u32x4_t g = *reinterpret_cast<const u32x4_t*>(norm_w + k);
        u32x4_t o;
        o.x = E::pack2(E::lo(g.x) * E::rnd(E::lo(v.x) * rs), E::hi(g.x) * E::rnd(E::hi(v.x) * rs));
        o.y = E::pack2(E::lo(g.y) * E::rnd(E::lo(v.y) * rs), E::hi(g.y) * E::rnd(E::hi(v.y) * rs));
        o.z = E::pack2(E::lo(g.z) * E::rnd(E::lo(v.z) * rs), E::hi(g.z) * E::rnd(E::hi(v.z) * rs));
        o.w = E::pack2(E::lo(g.w) * E::rnd(E::lo(v.w) * rs), E::hi(g.w) * E::rnd(E::hi(v.w) * rs));
        *reinterpret_cast<u32x4_t*>(dst + k) = o;
      }
    } else {
      for (int k = tid; k < Kp; k += kThreads) {
        uint16_t o = 0;
        if (k < K) {
          float v = E::rnd(E::val(src[k]) * rs);
          o = (uint16_t)E::bits(E::val(norm_w[k]) * v);
        }
        dst[k] = o;
      }
    }
  }
  __syncthreads();
}

// dot of NR weight rows against BATCH staged vectors; `first`/`step` give this thread's
// 8-element chunk walk (lane walk for a wave-owned row, thread walk for a block-owned row)
template <int DT, int NR, int BATCH>
__device__ __forceinline__ void dot_rows_vec8(const uint16_t* const (&wrow)[NR], const uint16_t* const (&xrow)[NR],
                                              int Kp, int K, int first, int step, float (&acc)[NR][BATCH]) {
  typedef E16<DT> E;
#pragma unroll 4
  for (int k = first; k < K; k += step) {
    u32x4_t w[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r) w[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(wrow[r] + k));
#pragma unroll
    for (int r = 0; r < NR; ++r) {
#pragma unroll
      for (int b = 0; b < BATCH; ++b) {
        u32x4_t xv = *reinterpret_cast<const u32x4_t*>(xrow[r] + b * Kp + k);
        acc[r][b] = E::dot8(w[r], xv, acc[r][b]);
      }
    }
  }
}

// the first PF chunks of every row, requested before the activations are staged so that the
// weight stream is already in flight while the block normalises / copies x
template <int NR, int PF>
__device__ __forceinline__ void prefetch_rows(const uint16_t* const (&wrow)[NR], int K, int first, int step,
                                              u32x4_t (&w)[NR][PF]) {
#pragma unroll
  for (int c = 0; c < PF; ++c) {
    const int k = first + c * step;
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      if (k < K) w[r][c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(wrow[r] + k));
      else w[r][c] = u32x4_t{0u, 0u, 0u, 0u};
    }
  }
}
template <int DT, int NR, int PF, int BATCH>
__device__ __forceinline__ void consume_rows(const u32x4_t (&w)[NR][PF], const uint16_t* const (&xrow)[NR], int Kp, int K,
                                             int first, int step, float (&acc)[NR][BATCH]) {
  typedef E16<DT> E;
#pragma unroll
  for (int c = 0; c < PF; ++c) {
    const int k = first + c * step;
    if (k < K) {
#pragma unroll
      for (int r = 0; r < NR; ++r)
#pragma unroll
        for (int b = 0; b < BATCH; ++b) {
          const u32x4_t xv = *reinterpret_cast<const u32x4_t*>(xrow[r] + b * Kp + k);
          acc[r][b] = E::dot8(w[r][c], xv, acc[r][b]);
        }
    }
  }
}

// fallback walk for rows whose start is not 16-byte aligned or whose length is not a multiple of 8
template <int DT, int NR, int BATCH>
__device__ __forceinline__ void dot_rows_scalar(const uint16_t* const (&wrow)[NR], const uint16_t* const (&xrow)[NR],
                                                int Kp, int K, int first, int step, float (&acc)[NR][BATCH]) {
  typedef E16<DT> E;
  for (int k = first; k < K; k += step) {
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      float w = E::val(wrow[r][k]);
#pragma unroll
      for (int b = 0; b < BATCH; ++b) acc[r][b] += w * E::val(xrow[r][b * Kp + k]);
    }
  }
}

// reduce acc over the owning group (wave or block); result valid in every thread
template <int NR, int BATCH, bool BLOCKROW>
__device__ __forceinline__ void reduce_acc(float (&acc)[NR][BATCH], float* red) {
#pragma unroll
  for (int r = 0; r < NR; ++r)
#pragma unroll
    for (int b = 0; b < BATCH; ++b) acc[r][b] = wave_sum(acc[r][b]);
  if (BLOCKROW) {
    const int wave = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) {
#pragma unroll
      for (int r = 0; r < NR; ++r)
#pragma unroll
        for (int b = 0; b < BATCH; ++b) red[(wave * NR + r) * BATCH + b] = acc[r][b];
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < NR; ++r)
#pragma unroll
      for (int b = 0; b < BATCH; ++b) {
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) t += red[(w * NR + r) * BATCH + b];
        acc[r][b] = t;
      }
  }
}

// ---------------------------------------------------------------------------------------
// y[b,n] = (res[b,n] +) bf16( W[n,:] . xn[b,:] (+ bias[n]) )
// ---------------------------------------------------------------------------------------
template <int DT, int BATCH, int ROWS, bool BLOCKROW, bool VEC>
__global__ __launch_bounds__(kThreads) void linear_kernel(LinearArgs a) {
  typedef E16<DT> E;
  extern __shared__ __align__(16) uint16_t smem[];
  __shared__ float red[kWaves * ROWS * BATCH > kWaves ? kWaves * ROWS * BATCH : kWaves];
  constexpr int PF = (8 / ROWS) > 1 ? (8 / ROWS) : 2;
  const int Kp = (a.K + 7) & ~7;
  const int b0 = blockIdx.y * BATCH;
  const int nb = min(BATCH, a.B - b0);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int group = BLOCKROW ? blockIdx.x : blockIdx.x * kWaves + wave;
  const int ngroups = BLOCKROW ? gridDim.x : gridDim.x * kWaves;
  const int first = (BLOCKROW ? tid : lane) * (VEC ? 8 : 1);
  const int step = (BLOCKROW ? kThreads : kWave) * (VEC ? 8 : 1);
  const int ngrp_rows = (a.N + ROWS - 1) / ROWS;

  const uint16_t* wrow[ROWS];
  const uint16_t* xrow[ROWS];
  int g = group;
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    wrow[r] = a.W + (int64_t)min(max(g, 0) * ROWS + r, a.N - 1) * a.ldw;
    xrow[r] = smem;
  }
  u32x4_t pf[ROWS][PF];
  bool have_pf = false;
  if (VEC && g < ngrp_rows) {
    prefetch_rows<ROWS, PF>(wrow, a.K, first, step, pf);
    have_pf = true;
  }
  stage_x<DT, BATCH>(a.x + (int64_t)b0 * a.ldx, a.ldx, nb, a.K, Kp, a.norm_w, a.eps, smem, red);

  // BLOCKROW needs every thread of the block in the loop (barriers inside reduce_acc)
  for (; g < ngrp_rows; g += ngroups) {
    const int n0 = g * ROWS;
    float acc[ROWS][BATCH];
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
#pragma unroll
      for (int b = 0; b < BATCH; ++b) acc[r][b] = 0.f;
    int kstart = first;
    if (have_pf) {
      consume_rows<DT, ROWS, PF, BATCH>(pf, xrow, Kp, a.K, first, step, acc);
      kstart = first + PF * step;
      have_pf = false;
    } else {
#pragma unroll
      for (int r = 0; r < ROWS; ++r) wrow[r] = a.W + (int64_t)min(n0 + r, a.N - 1) * a.ldw;
    }
    if (VEC) dot_rows_vec8<DT, ROWS, BATCH>(wrow, xrow, Kp, a.K, kstart, step, acc);
    else dot_rows_scalar<DT, ROWS, BATCH>(wrow, xrow, Kp, a.K, kstart, step, acc);
    reduce_acc<ROWS, BATCH, BLOCKROW>(acc, red);
    // epilogue: lane/thread (r*BATCH+b) stores one value
    const int who = BLOCKROW ? tid : lane;
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
#pragma unroll
      for (int b = 0; b < BATCH; ++b) {
        if (who == r * BATCH + b && n0 + r < a.N && b < nb) {
          const int n = n0 + r;
          float v = acc[r][b];
          if (a.bias) v += E::val(a.bias[n]);
          v = E::rnd(v);
          if (a.res) v = E::rnd(E::val(a.res[(int64_t)(b0 + b) * a.ldres + n]) + v);
          const uint16_t bits = (uint16_t)E::bits(v);
          a.y[(int64_t)(b0 + b) * a.ldy + n] = bits;
          if (a.positions) {               // the same value into the cache row of this token (uniform branch: a kernel argument)
            const int pos = a.positions[b0 + b];
            if (pos >= 0 && pos < a.app_S) {
#pragma unroll
              for (int i = 0; i < 2; ++i) {
                const int j = n - a.app_n0[i];
                if (a.app[i] && j >= 0 && j < a.app_n[i]) a.app[i][(int64_t)(b0 + b) * a.app_sb[i] + (int64_t)pos * a.app_ss[i] + j] = bits;
              }
            }
          }
        }
      }
  }
}

// ---------------------------------------------------------------------------------------
// h[b,n] = act( gate_u[n,:] . p[b, 0:R] , up_u[n,:] . p[b, up_off:up_off+R] )
//   mode 0 (chain of nn.Linear): g,u rounded to bf16, silu rounded, product rounded
//   mode 1 (fused-kernel rounding): h = bf16( silu(g32) * u32 )
// ---------------------------------------------------------------------------------------
template <int DT, int BATCH, int ROWS, bool VEC>
__global__ __launch_bounds__(kThreads) void swiglu_kernel(SwigluArgs a) {
  typedef E16<DT> E;
  extern __shared__ __align__(16) uint16_t smem[];
  __shared__ float red[kWaves];
  const int Kp = (a.R + 7) & ~7;
  const int b0 = blockIdx.y * BATCH;
  const int nb = min(BATCH, a.B - b0);
  constexpr int PF = (4 / ROWS) > 1 ? (4 / ROWS) : 2;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int group = blockIdx.x * kWaves + wave;
  const int ngroups = gridDim.x * kWaves;
  const int first = lane * (VEC ? 8 : 1), step = kWave * (VEC ? 8 : 1);
  const int ngrp_rows = (a.D + ROWS - 1) / ROWS;
  const uint16_t* wrow[2 * ROWS];
  const uint16_t* xrow[2 * ROWS];
  int g = group;
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int64_t off = (int64_t)min(g * ROWS + r, a.D - 1) * a.ldw;
    wrow[r] = a.gate_u + off;
    wrow[ROWS + r] = a.up_u + off;
    xrow[r] = smem;
    xrow[ROWS + r] = smem + BATCH * Kp;
  }
  u32x4_t pf[2 * ROWS][PF];
  bool have_pf = false;
  if (VEC && g < ngrp_rows) {
    prefetch_rows<2 * ROWS, PF>(wrow, a.R, first, step, pf);
    have_pf = true;
  }
  // two staged vectors per batch row: gate input then up input
  stage_x<DT, BATCH>(a.p + (int64_t)b0 * a.ldp, a.ldp, nb, a.R, Kp, nullptr, 0.f, smem, red);
  stage_x<DT, BATCH>(a.p + (int64_t)b0 * a.ldp + a.up_off, a.ldp, nb, a.R, Kp, nullptr, 0.f, smem + BATCH * Kp, red);

  for (; g < ngrp_rows; g += ngroups) {
    const int n0 = g * ROWS;
    float acc[2 * ROWS][BATCH];
#pragma unroll
    for (int r = 0; r < 2 * ROWS; ++r)
#pragma unroll
      for (int b = 0; b < BATCH; ++b) acc[r][b] = 0.f;
    int kstart = first;
    if (have_pf) {
      consume_rows<DT, 2 * ROWS, PF, BATCH>(pf, xrow, Kp, a.R, first, step, acc);
      kstart = first + PF * step;
      have_pf = false;
    } else {
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        const int64_t off = (int64_t)min(n0 + r, a.D - 1) * a.ldw;
        wrow[r] = a.gate_u + off;
        wrow[ROWS + r] = a.up_u + off;
      }
    }
    if (VEC) dot_rows_vec8<DT, 2 * ROWS, BATCH>(wrow, xrow, Kp, a.R, kstart, step, acc);
    else dot_rows_scalar<DT, 2 * ROWS, BATCH>(wrow, xrow, Kp, a.R, kstart, step, acc);
    reduce_acc<2 * ROWS, BATCH, false>(acc, red);
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
#pragma unroll
      for (int b = 0; b < BATCH; ++b) {
        if (lane == r * BATCH + b && n0 + r < a.D && b < nb) {
          float gv = acc[r][b], uv = acc[ROWS + r][b], hv;
          if (a.mode == 0) {
            gv = E::rnd(gv);
            uv = E::rnd(uv);
            hv = E::rnd(E::rnd(silu_f32(gv)) * uv);
          } else {
            hv = E::rnd((gv * (1.0f / (1.0f + expf(-gv)))) * uv);
          }
          a.h[(int64_t)(b0 + b) * a.ldh + n0 + r] = (uint16_t)E::bits(hv);
        }
      }
  }
}

// ---------------------------------------------------------------------------------------
// current-token q/k/v from rank coefficients, rotate-half RoPE on q and k, append k/v
//   p[b] = [Pq | Pk | Pv]; a work item is a row pair (d, d+Dh/2) of one head
// ---------------------------------------------------------------------------------------
template <int DT, int BATCH, int PAIRS, bool VEC>
__global__ __launch_bounds__(kThreads) void qkv_rope_append_kernel(QkvArgs a) {
  typedef E16<DT> E;
  extern __shared__ __align__(16) uint16_t smem[];
  __shared__ float red[kWaves];
  const int Rq8 = (a.Rq + 7) & ~7, Rk8 = (a.Rk + 7) & ~7, Rv8 = (a.Rv + 7) & ~7;
  const int b0 = blockIdx.y * BATCH;
  const int nb = min(BATCH, a.B - b0);
  uint16_t* xq = smem;
  uint16_t* xk = xq + BATCH * Rq8;
  uint16_t* xv = xk + BATCH * Rk8;
  const uint16_t* pb = a.p + (int64_t)b0 * a.ldp;
  stage_x<DT, BATCH>(pb, a.ldp, nb, a.Rq, Rq8, nullptr, 0.f, xq, red);
  stage_x<DT, BATCH>(pb + a.Rq, a.ldp, nb, a.Rk, Rk8, nullptr, 0.f, xk, red);
  stage_x<DT, BATCH>(pb + a.Rq + a.Rk, a.ldp, nb, a.Rv, Rv8, nullptr, 0.f, xv, red);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = a.Dh >> 1;
  const int npair_q = a.H * half, npair_kv = a.Hk * half;
  const int npairs = npair_q + 2 * npair_kv;
  const int group = blockIdx.x * kWaves + wave, ngroups = gridDim.x * kWaves;
  const int ngrp = (npairs + PAIRS - 1) / PAIRS;
  for (int g = group; g < ngrp; g += ngroups) {
    const uint16_t* wrow[2 * PAIRS];
    const uint16_t* xrow[2 * PAIRS];
    int kind[PAIRS], head[PAIRS], dd[PAIRS], Kp[PAIRS], K[PAIRS];
#pragma unroll
    for (int i = 0; i < PAIRS; ++i) {
      int pi = min(g * PAIRS + i, npairs - 1);
      if (pi < npair_q) {
        kind[i] = 0; head[i] = pi / half; dd[i] = pi % half;
        const uint16_t* base = a.q_u + (int64_t)(head[i] * a.Dh + dd[i]) * a.ldq;
        wrow[2 * i] = base; wrow[2 * i + 1] = base + (int64_t)half * a.ldq;
        xrow[2 * i] = xrow[2 * i + 1] = xq; Kp[i] = Rq8; K[i] = a.Rq;
      } else if (pi < npair_q + npair_kv) {
        pi -= npair_q;
        kind[i] = 1; head[i] = pi / half; dd[i] = pi % half;
        const uint16_t* base = a.k_u + (int64_t)(head[i] * a.Dh + dd[i]) * a.ldk;
        wrow[2 * i] = base; wrow[2 * i + 1] = base + (int64_t)half * a.ldk;
        xrow[2 * i] = xrow[2 * i + 1] = xk; Kp[i] = Rk8; K[i] = a.Rk;
      } else {
        pi -= npair_q + npair_kv;
        kind[i] = 2; head[i] = pi / half; dd[i] = pi % half;
        const uint16_t* base = a.v_u + (int64_t)(head[i] * a.Dh + dd[i]) * a.ldv;
        wrow[2 * i] = base; wrow[2 * i + 1] = base + (int64_t)half * a.ldv;
        xrow[2 * i] = xrow[2 * i + 1] = xv; Kp[i] = Rv8; K[i] = a.Rv;
      }
    }
    float acc[2 * PAIRS][BATCH];
#pragma unroll
    for (int r = 0; r < 2 * PAIRS; ++r)
#pragma unroll
      for (int b = 0; b < BATCH; ++b) acc[r][b] = 0.f;
    // ranks may differ between q/k/v, so each pair walks its own length
#pragma unroll
    for (int i = 0; i < PAIRS; ++i) {
      const uint16_t* w2[2] = {wrow[2 * i], wrow[2 * i + 1]};
      const uint16_t* x2[2] = {xrow[2 * i], xrow[2 * i + 1]};
      float acc2[2][BATCH];
#pragma unroll
      for (int b = 0; b < BATCH; ++b) acc2[0][b] = acc2[1][b] = 0.f;
      if (VEC) dot_rows_vec8<DT, 2, BATCH>(w2, x2, Kp[i], K[i], lane * 8, kWave * 8, acc2);
      else dot_rows_scalar<DT, 2, BATCH>(w2, x2, Kp[i], K[i], lane, kWave, acc2);
#pragma unroll
      for (int b = 0; b < BATCH; ++b) { acc[2 * i][b] = acc2[0][b]; acc[2 * i + 1][b] = acc2[1][b]; }
    }
    reduce_acc<2 * PAIRS, BATCH, false>(acc, red);
#pragma unroll
    for (int i = 0; i < PAIRS; ++i)
#pragma unroll
      for (int b = 0; b < BATCH; ++b) {
        if (lane == i * BATCH + b && g * PAIRS + i < npairs && b < nb) {
          const int bb = b0 + b;
          const int pos = a.positions[bb];
          float x0 = E::rnd(acc[2 * i][b]), x1 = E::rnd(acc[2 * i + 1][b]);
          if (kind[i] != 2 && a.cos) {
            // eager bf16 arithmetic: x0*c - x1*s and x1*c + x0*s, one rounding per op
            const int tp = min(max(pos, 0), a.rope_len - 1);
            const float c = E::val(a.cos[(int64_t)tp * half + dd[i]]);
            const float s = E::val(a.sin[(int64_t)tp * half + dd[i]]);
            const float r0 = E::rnd(E::rnd(x0 * c) - E::rnd(x1 * s));
            const float r1 = E::rnd(E::rnd(x1 * c) + E::rnd(x0 * s));
            x0 = r0; x1 = r1;
          }
          const uint16_t o0 = (uint16_t)E::bits(x0), o1 = (uint16_t)E::bits(x1);
          if (kind[i] == 0) {
            uint16_t* q = a.q_out + ((int64_t)bb * a.H + head[i]) * a.Dh + dd[i];
            q[0] = o0; q[half] = o1;
          } else if (pos >= 0 && pos < a.S) {
            uint16_t* base = (kind[i] == 1 ? a.k_cache : a.v_cache) + (int64_t)bb * a.sc_b + (int64_t)pos * a.sc_s +
                             (int64_t)head[i] * a.sc_h + dd[i];
            base[0] = o0; base[half] = o1;
          }
        }
      }
  }
}

// ---------------------------------------------------------------------------------------
// stand-alone RMSNorm (one block per row)
// ---------------------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(kThreads) void rmsnorm_kernel(const uint16_t* __restrict__ x, int64_t ldx,
                                                          const uint16_t* __restrict__ w, float eps,
                                                          uint16_t* __restrict__ y, int64_t ldy, int K) {
  typedef E16<DT> E;
  __shared__ float red[kWaves];
  const uint16_t* src = x + (int64_t)blockIdx.x * ldx;
  uint16_t* dst = y + (int64_t)blockIdx.x * ldy;
  float ss = 0.f;
  for (int k = threadIdx.x; k < K; k += kThreads) {
    float v = E::val(src[k]);
    ss += v * v;
  }
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int i = 0; i < kWaves; ++i) tot += red[i];
  const float rs = rsqrtf(tot / (float)K + eps);
  for (int k = threadIdx.x; k < K; k += kThreads) {
    float v = E::rnd(E::val(src[k]) * rs);
    dst[k] = (uint16_t)E::bits(E::val(w[k]) * v);
  }
}

// the same with 16-byte accesses and the row kept in registers between the two passes (K a multiple of 8, at most
// 8 * NC * kThreads, rows 16-byte aligned): a prompt of 512 rows x 4096 took 9.9 us with 2-byte accesses
template <int DT, int NC>
__global__ __launch_bounds__(kThreads) void rmsnorm_vec_kernel(const uint16_t* __restrict__ x, int64_t ldx,
                                                              const uint16_t* __restrict__ w, float eps,
                                                              uint16_t* __restrict__ y, int64_t ldy, int K) {
  typedef E16<DT> E;
  __shared__ float red[kWaves];
  const uint16_t* src = x + (int64_t)blockIdx.x * ldx;
  uint16_t* dst = y + (int64_t)blockIdx.x * ldy;
  const int nchunk = K >> 3;
  u32x4_t v[NC];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int ch = threadIdx.x + c * kThreads;
    v[c] = ch < nchunk ? *reinterpret_cast<const u32x4_t*>(src + ch * 8) : u32x4_t{0u, 0u, 0u, 0u};
    const uint32_t e[4] = {v[c].x, v[c].y, v[c].z, v[c].w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float a = E::lo(e[i]), b = E::hi(e[i]);
      ss += a * a;
      ss += b * b;
    }
  }
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int i = 0; i < kWaves; ++i) tot += red[i];
  const float rs = rsqrtf(tot / (float)K + eps);
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int ch = threadIdx.x + c * kThreads;
    if (ch >= nchunk) break;
    const u32x4_t wv = *reinterpret_cast<const u32x4_t*>(w + ch * 8);
    const uint32_t e[4] = {v[c].x, v[c].y, v[c].z, v[c].w}, g[4] = {wv.x, wv.y, wv.z, wv.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float a = E::rnd(E::lo(e[i]) * rs), b = E::rnd(E::hi(e[i]) * rs);
      o[i] = E::bits(E::lo(g[i]) * a) | (E::bits(E::hi(g[i]) * b) << 16);
    }
    *reinterpret_cast<u32x4_t*>(dst + ch * 8) = u32x4_t{o[0], o[1], o[2], o[3]};
  }
}

// ---------------------------------------------------------------------------------------
// host-side launchers
// ---------------------------------------------------------------------------------------
static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

#define FSVD_CHECK_LAUNCH(name)                                             \
  do {                                                                      \
    hipError_t e__ = hipGetLastError();                                     \
    if (e__ != hipSuccess) {                                                \
      set_last_error("%s: launch failed: %s", name, hipGetErrorString(e__)); \
      return kErrLaunch;                                                    \
    }                                                                       \
  } while (0)

template <int DT, int BATCH, bool VEC>
static int launch_linear_b(const LinearArgs& a, int cfg, hipStream_t st) {
  const int Kp = (a.K + 7) & ~7;
  const size_t smem = (size_t)BATCH * Kp * 2;
  const int nby = (a.B + BATCH - 1) / BATCH;
  // cfg: 0 auto, else (rows | blockrow<<8)
  int rows = cfg & 0xff;
  bool blockrow = (cfg >> 8) & 1;
  if (cfg == 0) {
    blockrow = a.K >= 8192;
    rows = (!blockrow && a.N >= 16384) ? 4 : 1;   // long outputs (lm_head) amortise the x reads over 4 rows
  }
  if (BATCH > 1 && rows > 2) rows = 2;
#define FSVD_LAUNCH_LIN(R, BR)                                                                   \
  {                                                                                              \
    const int groups = (a.N + R - 1) / R;                                                        \
    dim3 grid(BR ? groups : (groups + kWaves - 1) / kWaves, nby);                                \
    hipLaunchKernelGGL((linear_kernel<DT, BATCH, R, BR, VEC>), grid, dim3(kThreads), smem, st, a);   \
  }
  if (blockrow) {
    if (rows >= 2) FSVD_LAUNCH_LIN(2, true) else FSVD_LAUNCH_LIN(1, true)
  } else if (rows >= 4 && BATCH == 1) FSVD_LAUNCH_LIN(4, false)
  else if (rows >= 2) FSVD_LAUNCH_LIN(2, false)
  else FSVD_LAUNCH_LIN(1, false)
#undef FSVD_LAUNCH_LIN
  FSVD_CHECK_LAUNCH("fsvd_linear");
  return kOk;
}

template <int DT>
static int launch_linear_t(const LinearArgs& a, int cfg, hipStream_t st) {
  const bool vec = (a.K % 8 == 0) && (a.ldw % 8 == 0) && aligned16(a.W);
  const int batch = a.B >= 4 && a.K <= 16384 ? 4 : (a.B >= 2 ? 2 : 1);
  if (vec) {
    if (batch == 4) return launch_linear_b<DT, 4, true>(a, cfg, st);
    if (batch == 2) return launch_linear_b<DT, 2, true>(a, cfg, st);
    return launch_linear_b<DT, 1, true>(a, cfg, st);
  }
  if (batch == 4) return launch_linear_b<DT, 4, false>(a, cfg, st);
  if (batch == 2) return launch_linear_b<DT, 2, false>(a, cfg, st);
  return launch_linear_b<DT, 1, false>(a, cfg, st);
}

int launch_linear(const LinearArgs& a, int cfg, hipStream_t st) {
  if (a.B <= 0 || a.N <= 0 || a.K <= 0) { set_last_error("fsvd_linear: empty shape B=%d N=%d K=%d", a.B, a.N, a.K); return kErrBadShape; }
  if (a.dt != 0 && a.dt != 1) { set_last_error("fsvd_linear: dtype code %d (bf16 = 0 and fp16 = 1 are served)", a.dt); return kErrBadDtype; }
  if (cfg == 0 && mfma_linear_applies(a)) {
    if (a.positions) { set_last_error("fsvd_linear_rankkv_append: %d rows take the matrix-core kernels, which have no append epilogue (one or two rows)", a.B); return kErrBadShape; }
    return launch_linear_mfma(a, st);
  }
  if (a.K > 32768) { set_last_error("fsvd_linear: K=%d exceeds the 32768 LDS staging limit", a.K); return kErrBadShape; }
  return a.dt == 1 ? launch_linear_t<1>(a, cfg, st) : launch_linear_t<0>(a, cfg, st);
}

template <int DT, int BATCH, bool VEC>
static int launch_swiglu_b(const SwigluArgs& a, int cfg, hipStream_t st) {
  const int Kp = (a.R + 7) & ~7;
  const size_t smem = (size_t)2 * BATCH * Kp * 2;
  const int nby = (a.B + BATCH - 1) / BATCH;
  int rows = cfg & 0xff;
  if (rows == 0) rows = 1;
#define FSVD_LAUNCH_SW(R)                                                                  \
  {                                                                                        \
    const int groups = (a.D + R - 1) / R;                                                  \
    dim3 grid((groups + kWaves - 1) / kWaves, nby);                                        \
    hipLaunchKernelGGL((swiglu_kernel<DT, BATCH, R, VEC>), grid, dim3(kThreads), smem, st, a); \
  }
  if (rows >= 2 && BATCH <= 2) FSVD_LAUNCH_SW(2) else FSVD_LAUNCH_SW(1)
#undef FSVD_LAUNCH_SW
  FSVD_CHECK_LAUNCH("fsvd_swiglu_linear");
  return kOk;
}

template <int DT>
static int launch_swiglu_t(const SwigluArgs& a, int cfg, hipStream_t st) {
  const bool vec = (a.R % 8 == 0) && (a.ldw % 8 == 0) && aligned16(a.gate_u) && aligned16(a.up_u);
  const int batch = a.B >= 4 && a.R <= 4096 ? 4 : (a.B >= 2 ? 2 : 1);
  if (vec) {
    if (batch == 4) return launch_swiglu_b<DT, 4, true>(a, cfg, st);
    if (batch == 2) return launch_swiglu_b<DT, 2, true>(a, cfg, st);
    return launch_swiglu_b<DT, 1, true>(a, cfg, st);
  }
  if (batch == 4) return launch_swiglu_b<DT, 4, false>(a, cfg, st);
  if (batch == 2) return launch_swiglu_b<DT, 2, false>(a, cfg, st);
  return launch_swiglu_b<DT, 1, false>(a, cfg, st);
}

int launch_swiglu(const SwigluArgs& a, int cfg, hipStream_t st) {
  if (a.B <= 0 || a.D <= 0 || a.R <= 0) { set_last_error("fsvd_swiglu_linear: empty shape"); return kErrBadShape; }
  if (a.dt != 0 && a.dt != 1) { set_last_error("fsvd_swiglu_linear: dtype code %d (bf16 = 0 and fp16 = 1 are served)", a.dt); return kErrBadDtype; }
  if (cfg == 0 && mfma_swiglu_applies(a)) return launch_swiglu_mfma(a, st);
  if (a.R > 16384) { set_last_error("fsvd_swiglu_linear: R=%d exceeds 16384", a.R); return kErrBadShape; }
  return a.dt == 1 ? launch_swiglu_t<1>(a, cfg, st) : launch_swiglu_t<0>(a, cfg, st);
}

template <int DT, int BATCH, bool VEC>
static int launch_qkv_b(const QkvArgs& a, int cfg, hipStream_t st) {
  const int Rq8 = (a.Rq + 7) & ~7, Rk8 = (a.Rk + 7) & ~7, Rv8 = (a.Rv + 7) & ~7;
  const size_t smem = (size_t)BATCH * (Rq8 + Rk8 + Rv8) * 2;
  const int nby = (a.B + BATCH - 1) / BATCH;
  const int npairs = (a.H + 2 * a.Hk) * (a.Dh / 2);
  int pairs = cfg & 0xff;
  if (pairs == 0) pairs = 2;
#define FSVD_LAUNCH_QKV(P)                                                                          \
  {                                                                                                 \
    const int groups = (npairs + P - 1) / P;                                                        \
    dim3 grid((groups + kWaves - 1) / kWaves, nby);                                                 \
    hipLaunchKernelGGL((qkv_rope_append_kernel<DT, BATCH, P, VEC>), grid, dim3(kThreads), smem, st, a); \
  }
  if (pairs >= 2 && BATCH == 1) FSVD_LAUNCH_QKV(2) else FSVD_LAUNCH_QKV(1)
#undef FSVD_LAUNCH_QKV
  FSVD_CHECK_LAUNCH("fsvd_qkv_rope_append");
  return kOk;
}

static int check_qkv(const QkvArgs& a) {
  if (a.B <= 0 || a.H <= 0 || a.Hk <= 0 || a.Dh <= 0 || (a.Dh & 1) || a.Rq <= 0 || a.Rk <= 0 || a.Rv <= 0) {
    set_last_error("fsvd_qkv_rope_append: bad shape B=%d H=%d Hk=%d Dh=%d R=(%d,%d,%d)", a.B, a.H, a.Hk, a.Dh, a.Rq, a.Rk, a.Rv);
    return kErrBadShape;
  }
  if (a.Rq + a.Rk + a.Rv > 24576) { set_last_error("fsvd_qkv_rope_append: ranks too large for LDS staging"); return kErrBadShape; }
  if (a.dt != 0 && a.dt != 1) { set_last_error("fsvd_qkv_rope_append: dtype code %d (bf16 = 0 and fp16 = 1 are served)", a.dt); return kErrBadDtype; }
  return kOk;
}

template <int DT>
static int launch_qkv_t(const QkvArgs& a, int cfg, hipStream_t st) {
  const bool vec = (a.Rq % 8 == 0) && (a.Rk % 8 == 0) && (a.Rv % 8 == 0) && (a.ldq % 8 == 0) && (a.ldk % 8 == 0) &&
                   (a.ldv % 8 == 0) && aligned16(a.q_u) && aligned16(a.k_u) && aligned16(a.v_u);
  const int batch = a.B >= 4 && (a.Rq + a.Rk + a.Rv) <= 8192 ? 4 : (a.B >= 2 ? 2 : 1);
  if (vec) {
    if (batch == 4) return launch_qkv_b<DT, 4, true>(a, cfg, st);
    if (batch == 2) return launch_qkv_b<DT, 2, true>(a, cfg, st);
    return launch_qkv_b<DT, 1, true>(a, cfg, st);
  }
  if (batch == 4) return launch_qkv_b<DT, 4, false>(a, cfg, st);
  if (batch == 2) return launch_qkv_b<DT, 2, false>(a, cfg, st);
  return launch_qkv_b<DT, 1, false>(a, cfg, st);
}

int launch_qkv(const QkvArgs& a, int cfg, hipStream_t st) {
  const int rc = check_qkv(a);
  if (rc != kOk) return rc;
  return a.dt == 1 ? launch_qkv_t<1>(a, cfg, st) : launch_qkv_t<0>(a, cfg, st);
}

template <int DT>
static void launch_rmsnorm_t(const uint16_t* x, int64_t ldx, const uint16_t* w, float eps, uint16_t* y, int64_t ldy, int rows,
                             int K, hipStream_t st) {
  const auto al = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  const bool vec = (K % 8) == 0 && al(x) && al(w) && al(y) && (ldx % 8) == 0 && (ldy % 8) == 0;
  if (vec && K <= 8 * 2 * kThreads) hipLaunchKernelGGL((rmsnorm_vec_kernel<DT, 2>), dim3(rows), dim3(kThreads), 0, st, x, ldx, w, eps, y, ldy, K);
  else if (vec && K <= 8 * 8 * kThreads) hipLaunchKernelGGL((rmsnorm_vec_kernel<DT, 8>), dim3(rows), dim3(kThreads), 0, st, x, ldx, w, eps, y, ldy, K);
  else hipLaunchKernelGGL(rmsnorm_kernel<DT>, dim3(rows), dim3(kThreads), 0, st, x, ldx, w, eps, y, ldy, K);
}

int launch_rmsnorm(const uint16_t* x, int64_t ldx, const uint16_t* w, float eps, uint16_t* y, int64_t ldy, int rows,
                   int K, int dt, hipStream_t st) {
  if (rows <= 0 || K <= 0) { set_last_error("fsvd_rmsnorm: empty shape"); return kErrBadShape; }
  if (dt != 0 && dt != 1) { set_last_error("fsvd_rmsnorm: dtype code %d (bf16 = 0 and fp16 = 1 are served)", dt); return kErrBadDtype; }
  if (dt == 1) launch_rmsnorm_t<1>(x, ldx, w, eps, y, ldy, rows, K, st);
  else launch_rmsnorm_t<0>(x, ldx, w, eps, y, ldy, rows, K, st);
  FSVD_CHECK_LAUNCH("fsvd_rmsnorm");
  return kOk;
}

}  // namespace fsvd
