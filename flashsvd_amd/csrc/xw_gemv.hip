// y = x @ W for the reference's "input-major" operand layouts (W is [K, N], row k holds the
// contribution of input k to every output): the packed rank projection [d, Rq+Rk+Rv], the
// per-head bases [H, R, Dh], the prepacked flat bases [R, H*Dh] and the dual-split MLP operands
// GateU/UpU [R, D], DownV [D, R], DownU [R, Hd].
//
// A workgroup owns TN = 8*TX adjacent output columns and a slice of K.  Each thread keeps 8
// column accumulators in fp32, the 256/TX thread rows stride over the K slice (row segments of
// 16*TX bytes are read with one 16-byte load per lane), and the thread rows are folded through
// LDS.  With a K split the per-slice partials go to an fp32 workspace with write-through stores
// and the last workgroup to arrive for a tile adds them in slice order (deterministic), one
// output column per thread with sixteen shares in flight.  Aligned rows are read in whole trips
// of 8 (4) rows per thread row from two register sets, the next trip requested before the
// current one is multiplied; K slices are whole trips where K allows.
// Element types: bf16, fp16, fp32 (fp32 accumulate, one rounding at the store).
#include <hip/hip_fp16.h>
#include <type_traits>

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
  typedef u32x4_t Raw;                                   // eight elements as loaded
  static __device__ __forceinline__ Raw ldraw(const T* p) { return *reinterpret_cast<const u32x4_t*>(p); }
  static __device__ __forceinline__ void unpack(const Raw& r, float (&v)[8]) {
    v[0] = bf16_lo(r.x); v[1] = bf16_hi(r.x); v[2] = bf16_lo(r.y); v[3] = bf16_hi(r.y);
    v[4] = bf16_lo(r.z); v[5] = bf16_hi(r.z); v[6] = bf16_lo(r.w); v[7] = bf16_hi(r.w);
  }
};
template <> struct Elem<1> {  // fp16
  typedef uint16_t T;
  static __device__ __forceinline__ float ld(const T* p) { return __half2float(__ushort_as_half(*p)); }
  static __device__ __forceinline__ T cvt(float f) { return __half_as_ushort(__float2half_rn(f)); }
  static __device__ __forceinline__ float rnd(float f) { return __half2float(__float2half_rn(f)); }
  typedef u32x4_t Raw;
  static __device__ __forceinline__ Raw ldraw(const T* p) { return *reinterpret_cast<const u32x4_t*>(p); }
  static __device__ __forceinline__ void unpack(const Raw& r, float (&v)[8]) {
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
  typedef float f4 __attribute__((ext_vector_type(4)));
  struct Raw { f4 a, b; };
  static __device__ __forceinline__ Raw ldraw(const T* p) { return Raw{*reinterpret_cast<const f4*>(p), *reinterpret_cast<const f4*>(p + 4)}; }
  static __device__ __forceinline__ void unpack(const Raw& r, float (&v)[8]) {
    v[0] = r.a.x; v[1] = r.a.y; v[2] = r.a.z; v[3] = r.a.w; v[4] = r.b.x; v[5] = r.b.y; v[6] = r.b.z; v[7] = r.b.w;
  }
};

// epilogue of one output element: SwiGLU of the two products, or bias and rounding of one
template <int DT, bool DUAL>
__device__ __forceinline__ void xw_emit(const XwArgs& a, const XwProblem& P, int head, int row, int n, float v0, float v1) {
  typedef Elem<DT> E;
  typedef typename E::T T;
  float v;
  if (DUAL) {
    // h = dtype( silu(g) * u ) from the fp32 accumulators (g = x @ W, u = x2 @ W2)
    v = (v0 * (1.0f / (1.0f + expf(-v0)))) * v1;
  } else {
    v = v0;
    if (P.bias) {
      const float bv = E::ld(static_cast<const T*>(P.bias) + (int64_t)head * P.sbias_h + n);
      v = a.bias_post ? E::rnd(v) + bv : v + bv;   // bias_post: add after the rounding of the product
    }
  }
  if (a.out_fp32) static_cast<float*>(P.y)[(int64_t)row * P.sy_b + (int64_t)head * P.sy_h + n] = v;
  else static_cast<T*>(P.y)[(int64_t)row * P.sy_b + (int64_t)head * P.sy_h + n] = E::cvt(v);
}

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
  if (vec) {
    // aligned rows: UK rows per trip, every load of a trip requested before the first product.  Whole trips carry no
    // condition (a guard on a row's products makes the compiler sink that row's loads behind the guard, one round trip
    // per row); the rows left over are taken one at a time
    constexpr int UK = (DT == 2 || DUAL) ? 4 : 8;     // rows per trip (two matrices or 32-byte rows: half as many)
    const int64_t swk = P.sw_k;
    int k = k0 + ty;
    auto trip = [&](auto rows) {
      constexpr int U = decltype(rows)::value;
      typename E::Raw raw[U][NW];
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int w = 0; w < NW; ++w) raw[u][w] = E::ldraw(wbase[w] + (int64_t)(k + u * TY) * swk);
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int w = 0; w < NW; ++w) {
          float wv[8];
          E::unpack(raw[u][w], wv);
#pragma unroll
          for (int b = 0; b < BATCH; ++b) {
            const float xv = xs[w][b][k + u * TY - k0];
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[w][b][i] += xv * wv[i];
          }
        }
      k += TY * U;
    };
    // Whole trips, two register sets: the rows of the next trip are requested before the current ones are multiplied.
    // Nothing in the loop is conditional - a load whose use sits behind a condition is sunk behind it by the compiler,
    // a load under a condition makes it guard the registers with full waits: past the last trip the loads repeat the last
    // trip and their products are scaled by zero.
    {
      typedef typename E::Raw Raw;
      constexpr int S = TY * UK;
      const auto ld = [&](Raw (&r)[UK][NW], int kk) {
#pragma unroll
        for (int u = 0; u < UK; ++u)
#pragma unroll
          for (int w = 0; w < NW; ++w) r[u][w] = E::ldraw(wbase[w] + (int64_t)(kk + u * TY) * swk);
      };
      const auto fm = [&](const Raw (&r)[UK][NW], int kk, float scale) {
#pragma unroll
        for (int u = 0; u < UK; ++u)
#pragma unroll
          for (int w = 0; w < NW; ++w) {
            float wv[8];
            E::unpack(r[u][w], wv);
#pragma unroll
            for (int b = 0; b < BATCH; ++b) {
              const float xv = xs[w][b][kk + u * TY - k0] * scale;
#pragma unroll
              for (int i = 0; i < 8; ++i) acc[w][b][i] += xv * wv[i];
            }
          }
      };
      const int span = k1 - k - (UK - 1) * TY;             // > 0: at least one whole trip starts at k
      const int nT = span > 0 ? (span + S - 1) / S : 0;
      if (nT > 0) {
        Raw A[UK][NW], Bq[UK][NW];
        ld(A, k);
        for (int j = 0; j < nT; j += 2) {
          const int kb = k + min(j + 1, nT - 1) * S;
          ld(Bq, kb);
          fm(A, k + j * S, 1.0f);
          ld(A, k + min(j + 2, nT - 1) * S);
          fm(Bq, kb, j + 1 < nT ? 1.0f : 0.0f);
        }
        k += nT * S;
      }
    }
    if (k + (UK / 2 - 1) * TY < k1) trip(std::integral_constant<int, UK / 2>{});
    if (k + TY < k1) trip(std::integral_constant<int, 2>{});
    if (k < k1) trip(std::integral_constant<int, 1>{});
  } else if (ncol > 0) {
#pragma unroll 2
    for (int k = k0 + ty; k < k1; k += TY) {
      float wv[NW][8];
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const T* wp = wbase[w] + (int64_t)k * P.sw_k;
#pragma unroll
        for (int i = 0; i < 8; ++i) wv[w][i] = i < ncol ? E::ld(wp + i) : 0.f;
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
    if (tid == 0) __hip_atomic_store(&a.counters[tile_id], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // The last workgroup adds the shares with ALL its threads, one output column (of every matrix) per thread and SB
    // shares in flight at once: every load comes from beyond this XCD's L2, and with one share per round trip - or with
    // only the 8-column owners loading - the reduction was the longest part of a D-tiled product, whose shares number
    // K / 128.  The shares are added in split order.
    constexpr int SB = 16;
    for (int item = tid; item < BATCH * TN; item += kXwThreads) {
      const int b = item / TN, c = item - b * TN;
      const int n = n0 + c;
      float t[NW];
#pragma unroll
      for (int w = 0; w < NW; ++w) t[w] = 0.f;
      for (int s0 = 0; s0 < a.ksplit; s0 += SB) {
        float sh[SB][NW];
#pragma unroll
        for (int j = 0; j < SB; ++j) {
          const float* src = tile_ws + (int64_t)min(s0 + j, a.ksplit - 1) * (NW * BATCH * TN) + b * TN + c;
#pragma unroll
          for (int w = 0; w < NW; ++w) sh[j][w] = __hip_atomic_load(src + w * BATCH * TN, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int j = 0; j < SB; ++j)
#pragma unroll
          for (int w = 0; w < NW; ++w) t[w] += s0 + j < a.ksplit ? sh[j][w] : 0.f;
      }
      if (b < nb && n < P.N) xw_emit<DT, DUAL>(a, P, head, b0 + b, n, t[0], t[NW - 1]);
    }
    return;
  }

  if (ty != 0 || ncol <= 0) return;
#pragma unroll
  for (int b = 0; b < BATCH; ++b) {
    if (b >= nb) continue;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (i >= ncol) continue;
      xw_emit<DT, DUAL>(a, P, head, b0 + b, n0 + tx * 8 + i, tot[0][b][i], tot[NW - 1][b][i]);
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
      // about one workgroup per compute unit: every further split adds a share to the store -> count -> load chain at
      // the end, which costs more than the idle tail it fills (gate / up pair of the 7B MLP: 21.3 / 21.8 / 23.5 us at
      // 128 / 256 / 512 workgroups)
      while (base * ksplit < 256 && maxK / (ksplit * 2) >= 64) ksplit *= 2;
    }
    while ((maxK + ksplit - 1) / ksplit > kXwMaxKSlice) ++ksplit;
    // slices of whole trips of the row loop (64 rows: 8 thread rows x 8 rows per trip at the wide tile), as far as K allows
    if (ksplit > 1) {
      const int ksl = ((maxK + ksplit - 1) / ksplit + 63) / 64 * 64;
      ksplit = (maxK + ksl - 1) / ksl;
    }
    for (int i = 0; i < a.nprob; ++i) a.prob[i].kslice = ksplit > 1 ? ((maxK + ksplit - 1) / ksplit + 63) / 64 * 64 : a.prob[i].K;
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
