// Decode projections on group-wise int4 weights (1..4 activation rows): y = x . (s * (q - z))^T.
//
// Weights keep the layout of the quantised module (two columns per byte, even column in the low nibble;
// fp16 scale and int16 zero point per group of columns), so a row of K columns is K/2 bytes: a quarter of
// the 16-bit stream.  The kernel must not spend the saved bytes on unpacking, so no weight is ever
// converted to a float: OR-ing 0x4300 over a nibble n gives the bf16 bit pattern of 128 + n (0x4c00 over n << 6: the
// fp16 pattern of 16 + n), and V_DOT2_F32_{BF16,F16} multiplies two such weights with two activations of the same
// type straight from LDS.  With c = 128 or 16,
//     D_p = sum_k x_k * (c + q_k)     over the 32 columns of a 16-byte piece p,
//     X_p = sum_k x_k                 (computed once per workgroup when x is staged),
// the row is  y = sum_p s_g(p) * (D_p - (z_g(p) + c) * X_p): two shift/mask operations and one dot per two
// weights.  Activations are stored in LDS in the order the masks deliver the nibbles (columns 0,4 | 1,5 |
// 2,6 | 3,7 of every eight).  Eight lanes share 256 columns of a row, fold their partial sums with DPP and
// leave one value per 256 columns in LDS; a thread per output then adds the row's values in column order
// (deterministic) and applies the epilogue of the 16-bit kernels: bias, one rounding, residual, or SwiGLU.
#include "common.hpp"
#include "kernels.hpp"

namespace fsvd {

constexpr int kQT = 512;          // threads per workgroup
constexpr int kQUnroll = 4;       // pieces in flight per thread
typedef const __attribute__((address_space(1))) u32x4_t* q4_gptr_t;

__device__ __forceinline__ float half_bits_to_f32(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }

// sum over each aligned group of 8 lanes; every lane of the group gets the sum
__device__ __forceinline__ float row8_sum(float v) {
  v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_f32<0x141>(v);  // row_half_mirror
  return v;
}

// 32 weights (four dwords of nibbles) against 32 activations in the permuted LDS order
template <class E>
__device__ __forceinline__ float dot32_q4(const u32x4_t& q, const u32x4_t* xs) {
  float acc = 0.f;
  const uint32_t qd[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const u32x4_t xv = xs[j];
    const uint32_t d = qd[j];
    acc = E::dot2(E::template nib<0>(d), xv.x, acc);
    acc = E::dot2(E::template nib<4>(d), xv.y, acc);
    acc = E::dot2(E::template nib<8>(d), xv.z, acc);
    acc = E::dot2(E::template nib<12>(d), xv.w, acc);
  }
  return acc;
}

// NU pieces per thread of matrix m, starting at item i0: all loads first, then the products
template <class E, int BATCH, int NU>
__device__ __forceinline__ void q4_trip(const Q4Args& a, int m, int i0, int items, int r0, int PPR, int K, int nchunk,
                                        uint32_t ppr_magic, int gshift, const uint16_t* xs, const float* xsum, float* cp) {
  const int tid = threadIdx.x;
  const uint8_t* qw = a.qw[m];
  const uint16_t* sc = a.sc[m];
  const int16_t* zr = a.zr[m];
  u32x4_t q[NU];
  float s[NU], zz[NU];
  int piece[NU];
#pragma unroll
  for (int u = 0; u < NU; ++u) {
    const int i = min(i0 + u * kQT + tid, items - 1);
    const int row = (int)__umulhi((uint32_t)i, ppr_magic);
    piece[u] = i - row * PPR;
    const int64_t n = r0 + row;
    q[u] = __builtin_nontemporal_load((q4_gptr_t)(uintptr_t)(qw + n * a.ldq + (int64_t)piece[u] * 16));
    const int64_t gi = n * a.ldg + (piece[u] >> gshift);
    s[u] = half_bits_to_f32(sc[gi]);
    zz[u] = (float)((int)zr[gi] + E::nib_off);
  }
#pragma unroll
  for (int u = 0; u < NU; ++u) {
    const int i = i0 + u * kQT + tid;
#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
      const size_t xo = (size_t)m * BATCH + b;
      const float d = dot32_q4<E>(q[u], reinterpret_cast<const u32x4_t*>(xs + xo * K + (size_t)piece[u] * 32));
      const float part = row8_sum(s[u] * (d - zz[u] * xsum[xo * PPR + piece[u]]));
      if ((tid & 7) == 0 && i < items) cp[xo * nchunk + (i >> 3)] = part;
    }
  }
}

// BATCH activation rows, NMAT = 1 (linear) or 2 (gate and up of the SwiGLU, each with its own input)
template <int DT, int BATCH, int NMAT>
__global__ __launch_bounds__(kQT) void q4_linear_kernel(Q4Args a, int rows_per_wg, uint32_t ppr_magic, int gshift) {
  typedef E16<DT> E;
  extern __shared__ __align__(16) unsigned char q4_smem[];
  const int tid = threadIdx.x;
  const int K = a.K, PPR = K >> 5, CPR = PPR >> 3;
  const int r0 = blockIdx.x * rows_per_wg;
  const int nrows = min(rows_per_wg, a.N - r0);
  if (nrows <= 0) return;
  // LDS: activations (permuted), piece sums, chunk partials, reduction scratch
  uint16_t* xs = reinterpret_cast<uint16_t*>(q4_smem);                          // [NMAT][BATCH][K]
  float* xsum = reinterpret_cast<float*>(xs + (size_t)NMAT * BATCH * K);         // [NMAT][BATCH][PPR]
  float* cp = xsum + (size_t)NMAT * BATCH * PPR;                                // [NMAT][BATCH][rows_per_wg * CPR]
  float* red = cp + (size_t)NMAT * BATCH * rows_per_wg * CPR;                   // [8]
  const int nchunk = rows_per_wg * CPR;

  // ---- stage the activations -----------------------------------------------------------------------
  for (int m = 0; m < NMAT; ++m) {
    for (int b = 0; b < BATCH; ++b) {
      uint16_t* dst = xs + ((size_t)m * BATCH + b) * K;
      if (b >= a.B) {
        for (int k = tid * 8; k < K; k += kQT * 8) *reinterpret_cast<u32x4_t*>(dst + k) = u32x4_t{0u, 0u, 0u, 0u};
        continue;
      }
      const uint16_t* src = a.x + (int64_t)b * a.ldx + (m ? a.up_off : 0);
      float rs = 0.f;
      if (a.norm_w) {   // RMSNorm: w * round(x * rsqrt(mean(x^2) + eps)), sum in fp32
        float ss = 0.f;
        for (int k = tid * 8; k < K; k += kQT * 8) {
          const u32x4_t v = *reinterpret_cast<const u32x4_t*>(src + k);
          const float a0 = E::lo(v.x), a1 = E::hi(v.x), a2 = E::lo(v.y), a3 = E::hi(v.y);
          const float a4 = E::lo(v.z), a5 = E::hi(v.z), a6 = E::lo(v.w), a7 = E::hi(v.w);
          ss += ((a0 * a0 + a1 * a1) + (a2 * a2 + a3 * a3)) + ((a4 * a4 + a5 * a5) + (a6 * a6 + a7 * a7));
        }
        ss = wave_sum(ss);
        __syncthreads();
        if ((tid & 63) == 0) red[tid >> 6] = ss;
        __syncthreads();
        float tot = 0.f;
#pragma unroll
        for (int w = 0; w < kQT / 64; ++w) tot += red[w];
        rs = rsqrtf(tot / (float)K + a.eps);
      }
      for (int k = tid * 8; k < K; k += kQT * 8) {
        u32x4_t v = *reinterpret_cast<const u32x4_t*>(src + k);
        if (a.norm_w) {
          const u32x4_t g = *reinterpret_cast<const u32x4_t*>(a.norm_w + k);
          v.x = E::pack2(E::lo(g.x) * E::rnd(E::lo(v.x) * rs), E::hi(g.x) * E::rnd(E::hi(v.x) * rs));
          v.y = E::pack2(E::lo(g.y) * E::rnd(E::lo(v.y) * rs), E::hi(g.y) * E::rnd(E::hi(v.y) * rs));
          v.z = E::pack2(E::lo(g.z) * E::rnd(E::lo(v.z) * rs), E::hi(g.z) * E::rnd(E::hi(v.z) * rs));
          v.w = E::pack2(E::lo(g.w) * E::rnd(E::lo(v.w) * rs), E::hi(g.w) * E::rnd(E::hi(v.w) * rs));
        }
        // columns (0,1)(2,3)(4,5)(6,7) -> (0,4)(1,5)(2,6)(3,7)
        u32x4_t o;
        o.x = (v.x & 0xffffu) | (v.z << 16);
        o.y = (v.x >> 16) | (v.z & 0xffff0000u);
        o.z = (v.y & 0xffffu) | (v.w << 16);
        o.w = (v.y >> 16) | (v.w & 0xffff0000u);
        *reinterpret_cast<u32x4_t*>(dst + k) = o;
      }
    }
  }
  __syncthreads();
  for (int o = tid; o < NMAT * BATCH * PPR; o += kQT) {   // X_p: the 32 activations of a piece, added in storage order
    const u32x4_t* p = reinterpret_cast<const u32x4_t*>(xs + (size_t)o * 32);
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const u32x4_t v = p[j];
      s = E::dot2(E::one2, v.x, s);
      s = E::dot2(E::one2, v.y, s);
      s = E::dot2(E::one2, v.z, s);
      s = E::dot2(E::one2, v.w, s);
    }
    xsum[o] = s;
  }
  __syncthreads();

  // ---- stream the weights --------------------------------------------------------------------------
  const int items = nrows * PPR;
#pragma unroll
  for (int m = 0; m < NMAT; ++m) {
    int i0 = 0;
    for (; i0 + kQT * kQUnroll <= items; i0 += kQT * kQUnroll)     // full trips: kQUnroll pieces in flight per thread
      q4_trip<E, BATCH, kQUnroll>(a, m, i0, items, r0, PPR, K, nchunk, ppr_magic, gshift, xs, xsum, cp);
    for (; i0 < items; i0 += kQT)                                  // tail: one piece per thread
      q4_trip<E, BATCH, 1>(a, m, i0, items, r0, PPR, K, nchunk, ppr_magic, gshift, xs, xsum, cp);
  }
  __syncthreads();

  // ---- one thread per output: add the row's chunk values in column order, epilogue -------------------
  for (int o = tid; o < nrows * BATCH; o += kQT) {
    const int r = o / BATCH, b = o - r * BATCH;
    if (b >= a.B) continue;
    float v[NMAT];
#pragma unroll
    for (int m = 0; m < NMAT; ++m) {
      const float* c = cp + ((size_t)m * BATCH + b) * nchunk + (size_t)r * CPR;
      float t = 0.f;
      for (int j = 0; j < CPR; ++j) t += c[j];
      v[m] = t;
    }
    const int n = r0 + r;
    float out;
    if (NMAT == 2) {
      if (a.mode == 0) {
        const float g = E::rnd(v[0]), up = E::rnd(v[NMAT - 1]);
        out = E::rnd(E::rnd(silu_f32(g)) * up);
      } else {
        out = E::rnd((v[0] * (1.0f / (1.0f + expf(-v[0])))) * v[NMAT - 1]);
      }
    } else {
      float t = v[0];
      if (a.bias) t += E::val(a.bias[n]);
      out = E::rnd(t);
      if (a.res) out = E::rnd(E::val(a.res[(int64_t)b * a.ldres + n]) + out);
    }
    a.y[(int64_t)b * a.ldy + n] = (uint16_t)E::bits(out);
  }
}

// w[n, k] = round(s * (q - z)): the dense form of a quantised matrix (prefill runs on the matrix cores from it)
template <int DT>
__global__ __launch_bounds__(256) void q4_dequant_kernel(const uint8_t* __restrict__ qw, int64_t ldq, const uint16_t* __restrict__ sc,
                                                         const int16_t* __restrict__ zr, int64_t ldg, int group, uint16_t* __restrict__ w,
                                                         int64_t ldw, int N, int K) {
  typedef E16<DT> E;
  const int64_t bytes_per_row = (K + 1) / 2;
  const int64_t total = (int64_t)N * bytes_per_row;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t n = i / bytes_per_row;
    const int k = (int)(i - n * bytes_per_row) * 2;
    const uint32_t byte = qw[n * ldq + (k >> 1)];
    const int g0 = group > 0 ? k / group : 0, g1 = group > 0 ? (k + 1) / group : 0;
    w[n * ldw + k] = (uint16_t)E::bits(half_bits_to_f32(sc[n * ldg + g0]) * ((float)(int)(byte & 15u) - (float)zr[n * ldg + g0]));
    if (k + 1 < K)
      w[n * ldw + k + 1] = (uint16_t)E::bits(half_bits_to_f32(sc[n * ldg + g1]) * ((float)(int)(byte >> 4) - (float)zr[n * ldg + g1]));
  }
}

int launch_dequant_q4(const uint8_t* qw, int64_t ldq, const uint16_t* sc, const int16_t* zr, int64_t ldg, int group, uint16_t* w,
                      int64_t ldw, int N, int K, int dt, hipStream_t st) {
  if (dt != 0 && dt != 1) { set_last_error("fsvd_dequant_q4: dtype %d is neither bf16 (0) nor fp16 (1)", dt); return kErrBadDtype; }
  if (N <= 0 || K <= 0 || ldq < (K + 1) / 2 || ldw < K) { set_last_error("fsvd_dequant_q4: bad shape"); return kErrBadShape; }
  const int g = (group <= 0 || group >= K) ? 0 : group;
  if (g && ldg < (K + g - 1) / g) { set_last_error("fsvd_dequant_q4: scale rows shorter than the group count"); return kErrBadShape; }
  const int64_t total = (int64_t)N * ((K + 1) / 2);
  const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
  if (dt == 1) hipLaunchKernelGGL(q4_dequant_kernel<1>, dim3(blocks), dim3(256), 0, st, qw, ldq, sc, zr, ldg, g, w, ldw, N, K);
  else hipLaunchKernelGGL(q4_dequant_kernel<0>, dim3(blocks), dim3(256), 0, st, qw, ldq, sc, zr, ldg, g, w, ldw, N, K);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("fsvd_dequant_q4: launch failed: %s", hipGetErrorString(e)); return kErrLaunch; }
  return kOk;
}

static inline bool q4_al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

size_t q4_lds_bytes(int batch, int nmat, int K, int rows_per_wg) {
  const size_t ppr = (size_t)K / 32, cpr = ppr / 8;
  return (size_t)nmat * batch * K * 2 + (size_t)nmat * batch * ppr * 4 + (size_t)nmat * batch * rows_per_wg * cpr * 4 + 8 * 4;
}

template <int DT, int BATCH, int NMAT>
static int launch_q4_t(const Q4Args& a, int rows_per_wg, uint32_t magic, int gshift, size_t lds, hipStream_t st) {
  static size_t granted = 64 * 1024;   // dynamic LDS a kernel may use without asking
  if (lds > granted) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&q4_linear_kernel<DT, BATCH, NMAT>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) { set_last_error("fsvd_linear_q4: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e)); return kErrLaunch; }
    granted = lds;
  }
  const int nwg = (a.N + rows_per_wg - 1) / rows_per_wg;
  hipLaunchKernelGGL((q4_linear_kernel<DT, BATCH, NMAT>), dim3(nwg), dim3(kQT), lds, st, a, rows_per_wg, magic, gshift);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("fsvd_linear_q4: launch failed: %s", hipGetErrorString(e)); return kErrLaunch; }
  return kOk;
}

template <int DT>
static int launch_q4_batch(const Q4Args& a, int batch, int rows, uint32_t magic, int gshift, size_t lds, hipStream_t st) {
  if (a.nmat == 1) return batch == 1 ? launch_q4_t<DT, 1, 1>(a, rows, magic, gshift, lds, st)
                        : batch == 2 ? launch_q4_t<DT, 2, 1>(a, rows, magic, gshift, lds, st)
                                     : launch_q4_t<DT, 4, 1>(a, rows, magic, gshift, lds, st);
  return batch == 1 ? launch_q4_t<DT, 1, 2>(a, rows, magic, gshift, lds, st)
       : batch == 2 ? launch_q4_t<DT, 2, 2>(a, rows, magic, gshift, lds, st)
                    : launch_q4_t<DT, 4, 2>(a, rows, magic, gshift, lds, st);
}

int launch_linear_q4(const Q4Args& a0, hipStream_t st) {
  const char* fn = a0.nmat == 2 ? "fsvd_swiglu_linear_q4" : "fsvd_linear_q4";
  if (a0.dt != 0 && a0.dt != 1) { set_last_error("%s: dtype %d is neither bf16 (0) nor fp16 (1)", fn, a0.dt); return kErrBadDtype; }
  if (a0.B <= 0 || a0.N <= 0 || a0.K <= 0 || (a0.nmat != 1 && a0.nmat != 2)) { set_last_error("%s: empty problem", fn); return kErrBadShape; }
  if (a0.K % 256) { set_last_error("%s: K = %d is not a multiple of 256 (pad the factor)", fn, a0.K); return kErrBadShape; }
  int gshift;
  if (a0.group <= 0 || a0.group >= a0.K) {
    gshift = 31;                               // one group per row
  } else {
    if (a0.group < 32 || (a0.group & (a0.group - 1))) { set_last_error("%s: group size %d must be a power of two >= 32, or cover the row", fn, a0.group); return kErrBadShape; }
    gshift = __builtin_ctz((unsigned)a0.group) - 5;
    if (a0.ldg < (a0.K + a0.group - 1) / a0.group) { set_last_error("%s: scale rows shorter than the group count", fn); return kErrBadShape; }
  }
  if (a0.ldq < a0.K / 2 || (a0.ldq % 16) || (a0.ldx % 8) || (a0.up_off % 8)) { set_last_error("%s: row strides must keep 16-byte alignment", fn); return kErrBadAlign; }
  for (int m = 0; m < a0.nmat; ++m) {
    if (!a0.qw[m] || !a0.sc[m] || !a0.zr[m]) { set_last_error("%s: null weight, scale or zero pointer", fn); return kErrNullPtr; }
    if (!q4_al16(a0.qw[m])) { set_last_error("%s: packed weights must be 16-byte aligned", fn); return kErrBadAlign; }
  }
  if (!q4_al16(a0.x) || (a0.norm_w && !q4_al16(a0.norm_w))) { set_last_error("%s: activations / norm weight must be 16-byte aligned", fn); return kErrBadAlign; }
  const int ppr = a0.K / 32;
  // at least one piece per thread, at least twice as many weight bytes as staged activation bytes
  int rows = (a0.N + 511) / 512;
  rows = rows > (kQT + ppr - 1) / ppr ? rows : (kQT + ppr - 1) / ppr;
  rows = rows > 8 ? rows : 8;
  rows = rows < a0.N ? rows : a0.N;
  if ((int64_t)rows * ppr * ppr >= (1ll << 32)) { set_last_error("%s: row too long for the index arithmetic", fn); return kErrBadShape; }
  const uint32_t magic = 0xffffffffu / (uint32_t)ppr + 1u;
  for (int b0 = 0; b0 < a0.B; b0 += 4) {
    Q4Args a = a0;
    a.B = a0.B - b0 < 4 ? a0.B - b0 : 4;
    a.x = a0.x + (int64_t)b0 * a0.ldx;
    a.y = a0.y + (int64_t)b0 * a0.ldy;
    if (a0.res) a.res = a0.res + (int64_t)b0 * a0.ldres;
    const int batch = a.B == 1 ? 1 : (a.B == 2 ? 2 : 4);
    const size_t lds = q4_lds_bytes(batch, a.nmat, a.K, rows);
    if (lds > 160 * 1024) { set_last_error("%s: K = %d with %d rows needs %zu bytes of LDS", fn, a.K, a.B, lds); return kErrBadShape; }
    const int rc = a.dt == 1 ? launch_q4_batch<1>(a, batch, rows, magic, gshift, lds, st)
                             : launch_q4_batch<0>(a, batch, rows, magic, gshift, lds, st);
    if (rc != kOk) return rc;
  }
  return kOk;
}

}  // namespace fsvd
