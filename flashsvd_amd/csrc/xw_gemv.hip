// y = x @ W for the reference's "input-major" operand layouts (W is [K, N], row k holds the
// contribution of input k to every output): the packed rank projection [d, Rq+Rk+Rv], the
// per-head bases [H, R, Dh], the prepacked flat bases [R, H*Dh] and the dual-split MLP operands
// GateU/UpU [R, D], DownV [D, R], DownU [R, Hd].
//
// A workgroup owns TN = 8*TX adjacent output columns and a slice of K.  Each thread keeps 8
// column accumulators in fp32, the 256/TX thread rows stride over the K slice (row segments of
// 16*TX bytes are read with one 16-byte load per lane), and the thread rows are folded through
// LDS.  With a K split the per-slice partials go to an fp32 workspace with write-through stores
// and the last workgroup to arrive for a tile adds them in slice order (deterministic).
// Element types: bf16, fp16, fp32 (fp32 accumulate, one rounding at the store).
#include <hip/hip_fp16.h>

#include "common.hpp"
#include "kernels.hpp"

namespace fsvd {

constexpr int kXwThreads = 256;
constexpr int kXwMaxKSlice = 2048;

template <int DT> struct Elem;
template <> struct Elem<0> {  // bf16
  typedef uint16_t T;
  static __device__ __forceinline__ float ld(const T* p) { return bf16_bits_to_f32(*p); }
  static __device__ __forceinline__ T cvt(float f) { return (T)f32_to_bf16_bits(f); }
  static __device__ __forceinline__ float rnd(float f) { return round_bf16(f); }
  static __device__ __forceinline__ void ld8(const T* p, float (&v)[8]) {
    const u32x4_t r = *reinterpret_cast<const u32x4_t*>(p);
    v[0] = bf16_lo(r.x); v[1] = bf16_hi(r.x); v[2] = bf16_lo(r.y); v[3] = bf16_hi(r.y);
    v[4] = bf16_lo(r.z); v[5] = bf16_hi(r.z); v[6] = bf16_lo(r.w); v[7] = bf16_hi(r.w);
  }
};
template <> struct Elem<1> {  // fp16
  typedef uint16_t T;
  static __device__ __forceinline__ float ld(const T* p) { return __half2float(__ushort_as_half(*p)); }
  static __device__ __forceinline__ T cvt(float f) { return __half_as_ushort(__float2half_rn(f)); }
  static __device__ __forceinline__ float rnd(float f) { return __half2float(__float2half_rn(f)); }
  static __device__ __forceinline__ void ld8(const T* p, float (&v)[8]) {
    const u32x4_t r = *reinterpret_cast<const u32x4_t*>(p);
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __half2float(__ushort_as_half((unsigned short)(w[i] & 0xffffu)));
      v[2 * i + 1] = __half2float(__ushort_as_half((unsigned short)(w[i] >> 16)));
    }
  }
};
template <> struct Elem<2> {  // fp32
  typedef float T;
  static __device__ __forceinline__ float ld(const T* p) { return *p; }
  static __device__ __forceinline__ T cvt(float f) { return f; }
  static __device__ __forceinline__ float rnd(float f) { return f; }
  static __device__ __forceinline__ void ld8(const T* p, float (&v)[8]) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    const f4 a = *reinterpret_cast<const f4*>(p), b = *reinterpret_cast<const f4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
};

template <int DT, int TX, int BATCH, bool DUAL>
__global__ __launch_bounds__(kXwThreads) void xw_gemv_kernel(XwArgs a) {
  typedef Elem<DT> E;
  typedef typename E::T T;
  constexpr int TY = kXwThreads / TX;
  constexpr int TN = TX * 8;
  constexpr int NW = DUAL ? 2 : 1;
  __shared__ float xs[NW][BATCH][kXwMaxKSlice];
  __shared__ float red[TY][TN + 4];
  __shared__ int last_flag;

  // which problem / head does this z index belong to
  int z = blockIdx.z, pi = 0;
  while (pi + 1 < a.nprob && z >= a.prob[pi].heads) { z -= a.prob[pi].heads; ++pi; }
  const XwProblem& P = a.prob[pi];
  const int head = z;
  const int ntile = blockIdx.x % a.ntiles_n;
  const int btile = blockIdx.x / a.ntiles_n;
  const int ks = blockIdx.y;
  const int n0 = ntile * TN;
  if (n0 >= P.N) return;   // problems may have fewer column tiles than the grid
  const int b0 = btile * BATCH;
  const int nb = min(BATCH, a.B - b0);
  const int kslice = P.kslice;
  const int k0 = ks * kslice;
  const int k1 = min(P.K, k0 + kslice);
  const int tid = threadIdx.x, tx = tid % TX, ty = tid / TX;
  const int ncol = min(8, P.N - (n0 + tx * 8));   // <= 0: thread has no columns

  // stage x[b, k0:k1) as fp32
  for (int w = 0; w < NW; ++w) {
    const T* xb = static_cast<const T*>(w == 0 ? P.x : P.x2) + (int64_t)head * P.sx_h;
    for (int b = 0; b < BATCH; ++b)
      for (int k = tid; k < k1 - k0; k += kXwThreads)
      {
        const int64_t off = (int64_t)(b0 + b) * P.sx_b + (int64_t)(k0 + k) * P.sx_k;
        float v = 0.f;
        if (b < nb) v = a.x_fp32 ? reinterpret_cast<const float*>(w == 0 ? P.x : P.x2)[(int64_t)head * P.sx_h + off] : E::ld(xb + off);
        xs[w][b][k] = a.x_round ? E::rnd(v) : v;
      }
  }
  __syncthreads();

  float acc[NW][BATCH][8];
#pragma unroll
  for (int w = 0; w < NW; ++w)
#pragma unroll
    for (int b = 0; b < BATCH; ++b)
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[w][b][i] = 0.f;

  const bool vec = P.vec && ncol == 8;
  const T* wbase[NW];
  wbase[0] = static_cast<const T*>(P.W) + (int64_t)head * P.sw_h + n0 + tx * 8;
  if (DUAL) wbase[NW - 1] = static_cast<const T*>(P.W2) + (int64_t)head * P.sw_h + n0 + tx * 8;
  if (ncol > 0) {
#pragma unroll 4
    for (int k = k0 + ty; k < k1; k += TY) {
      float wv[NW][8];
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const T* wp = wbase[w] + (int64_t)k * P.sw_k;
        if (vec) E::ld8(wp, wv[w]);
        else {
#pragma unroll
          for (int i = 0; i < 8; ++i) wv[w][i] = i < ncol ? E::ld(wp + i) : 0.f;
        }
      }
#pragma unroll
      for (int w = 0; w < NW; ++w)
#pragma unroll
        for (int b = 0; b < BATCH; ++b) {
          const float xv = xs[w][b][k - k0];
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[w][b][i] += xv * wv[w][i];
        }
    }
  }

  // fold the TY thread rows; thread (ty==0, tx) ends up owning 8 columns per (w, b)
  float tot[NW][BATCH][8];
#pragma unroll
  for (int w = 0; w < NW; ++w)
#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
      __syncthreads();
#pragma unroll
      for (int i = 0; i < 8; ++i) red[ty][tx * 8 + i] = acc[w][b][i];
      __syncthreads();
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float t = 0.f;
        if (ty == 0) {
#pragma unroll
          for (int r = 0; r < TY; ++r) t += red[r][tx * 8 + i];
        }
        tot[w][b][i] = t;
      }
    }

  if (a.ksplit > 1) {
    // partials: [tile][slice][w][b][TN] fp32, write-through; last arrival adds them in slice order
    const int64_t tile_id = ((int64_t)blockIdx.z * gridDim.x + blockIdx.x);
    float* tile_ws = a.ws + tile_id * a.ksplit * (NW * BATCH * TN);
    if (ty == 0) {
      float* mine = tile_ws + (int64_t)ks * (NW * BATCH * TN);
#pragma unroll
      for (int w = 0; w < NW; ++w)
#pragma unroll
        for (int b = 0; b < BATCH; ++b)
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            float v = tot[w][b][i];
            if (a.round_partials) v = E::rnd(v);
            __hip_atomic_store(mine + (w * BATCH + b) * TN + tx * 8 + i, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
    }
    wait_stores_acked();
    __syncthreads();
    if (tid == 0) {
      const int old = __hip_atomic_fetch_add(&a.counters[tile_id], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      last_flag = (old == a.ksplit - 1);
    }
    __syncthreads();
    if (!last_flag) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    if (ty == 0) {
#pragma unroll
      for (int w = 0; w < NW; ++w)
#pragma unroll
        for (int b = 0; b < BATCH; ++b)
#pragma unroll
          for (int i = 0; i < 8; ++i) tot[w][b][i] = 0.f;
      // one share at a time, all of its words in flight together (every load comes from beyond this XCD's L2; with the
      // shares as the inner loop each word cost a round trip of its own); the shares are added in split order
      for (int s = 0; s < a.ksplit; ++s) {
        float sh[NW][BATCH][8];
#pragma unroll
        for (int w = 0; w < NW; ++w)
#pragma unroll
          for (int b = 0; b < BATCH; ++b)
#pragma unroll
            for (int i = 0; i < 8; ++i)
              sh[w][b][i] = __hip_atomic_load(tile_ws + (int64_t)s * (NW * BATCH * TN) + (w * BATCH + b) * TN + tx * 8 + i,
                                              __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int w = 0; w < NW; ++w)
#pragma unroll
          for (int b = 0; b < BATCH; ++b)
#pragma unroll
            for (int i = 0; i < 8; ++i) tot[w][b][i] += sh[w][b][i];
      }
    }
    if (tid == 0) __hip_atomic_store(&a.counters[tile_id], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  if (ty != 0 || ncol <= 0) return;
#pragma unroll
  for (int b = 0; b < BATCH; ++b) {
    if (b >= nb) continue;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (i >= ncol) continue;
      const int n = n0 + tx * 8 + i;
      float v;
      if (DUAL) {
        // h = dtype( silu(g) * u ) from the fp32 accumulators (g = x @ W, u = x2 @ W2)
        const float g = tot[0][b][i], u = tot[NW - 1][b][i];
        v = (g * (1.0f / (1.0f + expf(-g)))) * u;
      } else {
        v = tot[0][b][i];
        if (P.bias) {
          const float bv = E::ld(static_cast<const T*>(P.bias) + (int64_t)head * P.sbias_h + n);
          v = a.bias_post ? E::rnd(v) + bv : v + bv;   // bias_post: add after the rounding of the product
        }
      }
      if (a.out_fp32) static_cast<float*>(P.y)[(int64_t)(b0 + b) * P.sy_b + (int64_t)head * P.sy_h + n] = v;
      else static_cast<T*>(P.y)[(int64_t)(b0 + b) * P.sy_b + (int64_t)head * P.sy_h + n] = E::cvt(v);
    }
  }
}

size_t xw_num_tiles(const XwArgs& a) { return a.ksplit > 1 ? (size_t)a.grid_x * a.grid_z : 0; }
size_t xw_partial_floats(const XwArgs& a, int tn, int batch_tile) {
  if (a.ksplit <= 1) return 0;
  return (size_t)a.grid_x * a.grid_z * a.ksplit * (size_t)((a.dual ? 2 : 1) * batch_tile * tn);
}

template <int DT, int TX, bool DUAL>
static void launch_xw_b(const XwArgs& a, int batch_tile, dim3 grid, hipStream_t st) {
  if (batch_tile == 4) hipLaunchKernelGGL((xw_gemv_kernel<DT, TX, 4, DUAL>), grid, dim3(kXwThreads), 0, st, a);
  else if (batch_tile == 2) hipLaunchKernelGGL((xw_gemv_kernel<DT, TX, 2, DUAL>), grid, dim3(kXwThreads), 0, st, a);
  else hipLaunchKernelGGL((xw_gemv_kernel<DT, TX, 1, DUAL>), grid, dim3(kXwThreads), 0, st, a);
}

template <int DT>
static void launch_xw_dt(const XwArgs& a, int tx, int batch_tile, dim3 grid, hipStream_t st) {
  if (a.dual) {
    if (tx == 16) launch_xw_b<DT, 16, true>(a, batch_tile, grid, st);
    else launch_xw_b<DT, 32, true>(a, batch_tile, grid, st);
  } else {
    if (tx == 16) launch_xw_b<DT, 16, false>(a, batch_tile, grid, st);
    else launch_xw_b<DT, 32, false>(a, batch_tile, grid, st);
  }
}

// Fills the launch geometry of `a` (tile width, K split, grid) for its problems.  `want_ksplit`
// = 0 picks a split that gives a few hundred workgroups; a caller that needs a fixed slice size
// (the D-tile of the dual-split MLP) passes kslice_fixed.
int plan_xw(XwArgs& a, int dtype, int want_ksplit, int kslice_fixed, int* tx_out, int* batch_tile_out) {
  if (a.nprob < 1 || a.nprob > 3 || a.B <= 0) { set_last_error("xw_gemv: bad problem count / batch"); return kErrBadShape; }
  int maxN = 0, maxK = 0, heads = 0;
  for (int i = 0; i < a.nprob; ++i) {
    XwProblem& P = a.prob[i];
    if (P.K <= 0 || P.N <= 0 || P.heads <= 0) { set_last_error("xw_gemv: empty problem K=%d N=%d heads=%d", P.K, P.N, P.heads); return kErrBadShape; }
    maxN = max(maxN, P.N); maxK = max(maxK, P.K); heads += P.heads;
    const int esz = dtype == 2 ? 4 : 2;
    const int per16 = 16 / esz;   // elements per 16 bytes
    P.vec = (P.sw_k % per16 == 0) && (P.sw_h % per16 == 0) && ((reinterpret_cast<uintptr_t>(P.W) & 15) == 0) &&
            (!a.dual || (reinterpret_cast<uintptr_t>(P.W2) & 15) == 0);
  }
  const int tx = maxN <= 128 ? 16 : 32;
  const int tn = tx * 8;
  const int batch_tile = a.dual ? (a.B >= 2 ? 2 : 1) : (a.B >= 4 ? 4 : (a.B >= 2 ? 2 : 1));
  a.ntiles_n = (maxN + tn - 1) / tn;
  const int nbt = (a.B + batch_tile - 1) / batch_tile;
  int ksplit;
  if (kslice_fixed > 0) {
    if (kslice_fixed > kXwMaxKSlice) { set_last_error("xw_gemv: K slice %d exceeds %d", kslice_fixed, kXwMaxKSlice); return kErrBadShape; }
    ksplit = (maxK + kslice_fixed - 1) / kslice_fixed;
    for (int i = 0; i < a.nprob; ++i) a.prob[i].kslice = kslice_fixed;
  } else {
    ksplit = want_ksplit > 0 ? want_ksplit : 1;
    if (want_ksplit <= 0) {
      const int base = a.ntiles_n * nbt * heads;
      while (base * ksplit < 512 && maxK / (ksplit * 2) >= 64) ksplit *= 2;
    }
    while ((maxK + ksplit - 1) / ksplit > kXwMaxKSlice) ++ksplit;
    for (int i = 0; i < a.nprob; ++i) a.prob[i].kslice = (a.prob[i].K + ksplit - 1) / ksplit;
  }
  a.ksplit = ksplit;
  a.grid_x = a.ntiles_n * nbt;
  a.grid_z = heads;
  *tx_out = tx;
  *batch_tile_out = batch_tile;
  return kOk;
}

int launch_xw(XwArgs& a, int dtype, int tx, int batch_tile, int32_t* counters, float* partials, hipStream_t st) {
  if (dtype < 0 || dtype > 2) { set_last_error("xw_gemv: dtype code %d not in {0,1,2}", dtype); return kErrBadDtype; }
  if (a.ksplit > 1 && (!counters || !partials)) { set_last_error("xw_gemv: split-K needs a workspace"); return kErrWorkspace; }
  a.counters = counters;
  a.ws = partials;
  dim3 grid(a.grid_x, a.ksplit, a.grid_z);
  if (dtype == 0) launch_xw_dt<0>(a, tx, batch_tile, grid, st);
  else if (dtype == 1) launch_xw_dt<1>(a, tx, batch_tile, grid, st);
  else launch_xw_dt<2>(a, tx, batch_tile, grid, st);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("xw_gemv: launch failed: %s", hipGetErrorString(e)); return kErrLaunch; }
  return kOk;
}

}  // namespace fsvd
