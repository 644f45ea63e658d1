// extern "C" surface of libflashsvd_hip: argument checks, then the launchers.
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <algorithm>
#include <mutex>

#include "../../include/flashsvd_hip.h"
#include "common.hpp"
#include "kernels.hpp"

namespace fsvd {
static thread_local char g_last_error[512] = "";
void set_last_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
}
}  // namespace fsvd

namespace fsvd {
// scratch registered by the caller for the K-split projections, one per device
constexpr int kMaxDevices = 16;
constexpr size_t kWsCounterBytes = 64 * 1024;
static SplitWorkspace g_split_ws[kMaxDevices] = {};
SplitWorkspace split_workspace() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return SplitWorkspace{nullptr, 0, nullptr, 0};
  return g_split_ws[dev];
}
__global__ void ws_clear_kernel(int32_t* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}
}  // namespace fsvd

using namespace fsvd;

#define FSVD_REQUIRE_PTR(p, fn)                             \
  if ((p) == nullptr) {                                     \
    set_last_error("%s: argument %s is NULL", fn, #p);      \
    return kErrNullPtr;                                     \
  }

static inline const uint16_t* cu16(const void* p) { return static_cast<const uint16_t*>(p); }
static inline uint16_t* u16(void* p) { return static_cast<uint16_t*>(p); }

extern "C" {

int fsvd_version(void) { return 102; }
const char* fsvd_last_error(void) { return g_last_error; }

int fsvd_set_workspace(void* ws, size_t bytes, void* stream) {
  const char* fn = "fsvd_set_workspace";
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) { set_last_error("%s: no current device", fn); return kErrLaunch; }
  if (ws == nullptr) { g_split_ws[dev] = SplitWorkspace{nullptr, 0, nullptr, 0}; return kOk; }
  if ((reinterpret_cast<uintptr_t>(ws) & 255) != 0) { set_last_error("%s: buffer must be 256-byte aligned", fn); return kErrBadAlign; }
  if (bytes < (size_t)1 << 20) { set_last_error("%s: %zu bytes is too small (1 MiB at least)", fn, bytes); return kErrBadShape; }
  const int ncount = (int)(kWsCounterBytes / sizeof(int32_t));
  hipLaunchKernelGGL(ws_clear_kernel, dim3((ncount + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<int32_t*>(ws), ncount);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("%s: launch failed: %s", fn, hipGetErrorString(e)); return kErrLaunch; }
  g_split_ws[dev] = SplitWorkspace{reinterpret_cast<float*>(static_cast<char*>(ws) + kWsCounterBytes), (bytes - kWsCounterBytes) / sizeof(float),
                                   static_cast<int32_t*>(ws), ncount};
  return kOk;
}

int fsvd_linear(const void* x, int64_t ldx, const void* W, int64_t ldw, const void* bias, const void* norm_w, float eps,
                const void* res, int64_t ldres, void* y, int64_t ldy, int B, int N, int K, int cfg, int dtype, void* stream) {
  FSVD_REQUIRE_PTR(x, "fsvd_linear"); FSVD_REQUIRE_PTR(W, "fsvd_linear"); FSVD_REQUIRE_PTR(y, "fsvd_linear");
  if (ldx < K || ldw < K || ldy < N || (res && ldres < N)) {
    set_last_error("fsvd_linear: leading dimension smaller than the row (ldx=%lld ldw=%lld ldy=%lld ldres=%lld K=%d N=%d)",
                   (long long)ldx, (long long)ldw, (long long)ldy, (long long)ldres, K, N);
    return kErrBadShape;
  }
  LinearArgs a{cu16(x), ldx, cu16(W), ldw, cu16(bias), cu16(norm_w), eps, cu16(res), ldres, u16(y), ldy, B, N, K, dtype};
  return launch_linear(a, cfg, static_cast<hipStream_t>(stream));
}

int fsvd_linear_rankkv_append(const void* x, int64_t ldx, const void* W, int64_t ldw, const void* norm_w, float eps, void* y, int64_t ldy,
                              int B, int Rq, int Rk, int Rv, int K, void* pk_cache, int64_t spk_b, int64_t spk_s, void* pv_cache,
                              int64_t spv_b, int64_t spv_s, const int32_t* positions, int S, int dtype, void* stream) {
  const char* fn = "fsvd_linear_rankkv_append";
  FSVD_REQUIRE_PTR(x, fn); FSVD_REQUIRE_PTR(W, fn); FSVD_REQUIRE_PTR(y, fn); FSVD_REQUIRE_PTR(pk_cache, fn); FSVD_REQUIRE_PTR(pv_cache, fn);
  FSVD_REQUIRE_PTR(positions, fn);
  if (B <= 0 || B > 2) { set_last_error("%s: %d rows (one or two: more rows take fsvd_linear and fsvd_rankkv_append)", fn, B); return kErrBadShape; }
  if (Rq < 0 || Rk <= 0 || Rv <= 0 || S <= 0) { set_last_error("%s: bad ranks / cache length (Rq=%d Rk=%d Rv=%d S=%d)", fn, Rq, Rk, Rv, S); return kErrBadShape; }
  const int N = Rq + Rk + Rv;
  if (ldx < K || ldw < K || ldy < N || spk_s < Rk || spv_s < Rv) { set_last_error("%s: a leading dimension is smaller than its row", fn); return kErrBadShape; }
  LinearArgs a{cu16(x), ldx, cu16(W), ldw, nullptr, cu16(norm_w), eps, nullptr, 0, u16(y), ldy, B, N, K, dtype};
  a.positions = positions;
  a.app[0] = u16(pk_cache); a.app_sb[0] = spk_b; a.app_ss[0] = spk_s; a.app_n0[0] = Rq; a.app_n[0] = Rk;
  a.app[1] = u16(pv_cache); a.app_sb[1] = spv_b; a.app_ss[1] = spv_s; a.app_n0[1] = Rq + Rk; a.app_n[1] = Rv;
  a.app_S = S;
  return launch_linear(a, 0, static_cast<hipStream_t>(stream));
}

int fsvd_swiglu_linear(const void* p, int64_t ldp, int64_t up_off, const void* gate_u, const void* up_u, int64_t ldw,
                       void* h, int64_t ldh, int B, int D, int R, int mode, int cfg, int dtype, void* stream) {
  FSVD_REQUIRE_PTR(p, "fsvd_swiglu_linear"); FSVD_REQUIRE_PTR(gate_u, "fsvd_swiglu_linear");
  FSVD_REQUIRE_PTR(up_u, "fsvd_swiglu_linear"); FSVD_REQUIRE_PTR(h, "fsvd_swiglu_linear");
  if (up_off < 0 || ldp < up_off + R || ldw < R || ldh < D || (mode != 0 && mode != 1)) {
    set_last_error("fsvd_swiglu_linear: inconsistent layout (ldp=%lld up_off=%lld R=%d ldw=%lld ldh=%lld D=%d mode=%d)",
                   (long long)ldp, (long long)up_off, R, (long long)ldw, (long long)ldh, D, mode);
    return kErrBadShape;
  }
  SwigluArgs a{cu16(p), ldp, up_off, cu16(gate_u), cu16(up_u), ldw, u16(h), ldh, B, D, R, mode, dtype};
  return launch_swiglu(a, cfg, static_cast<hipStream_t>(stream));
}

int fsvd_linear_q4(const void* x, int64_t ldx, const void* qweight, int64_t ldq, const void* scales, const void* zeros,
                   int64_t ldg, int group_size, const void* bias, const void* norm_w, float eps, const void* res,
                   int64_t ldres, void* y, int64_t ldy, int B, int N, int K, int dtype, void* stream) {
  const char* fn = "fsvd_linear_q4";
  FSVD_REQUIRE_PTR(x, fn); FSVD_REQUIRE_PTR(qweight, fn); FSVD_REQUIRE_PTR(scales, fn); FSVD_REQUIRE_PTR(zeros, fn);
  FSVD_REQUIRE_PTR(y, fn);
  if (ldx < K || ldy < N || (res && ldres < N)) { set_last_error("%s: leading dimension smaller than the row", fn); return kErrBadShape; }
  Q4Args a{cu16(x), ldx, 0, {static_cast<const uint8_t*>(qweight), nullptr}, ldq, {cu16(scales), nullptr},
           {static_cast<const int16_t*>(zeros), nullptr}, ldg, group_size, cu16(bias), cu16(norm_w), eps, cu16(res), ldres,
           u16(y), ldy, B, N, K, 1, 0, dtype};
  return launch_linear_q4(a, static_cast<hipStream_t>(stream));
}

int fsvd_dequant_q4(const void* qweight, int64_t ldq, const void* scales, const void* zeros, int64_t ldg, int group_size,
                    void* w, int64_t ldw, int N, int K, int dtype, void* stream) {
  const char* fn = "fsvd_dequant_q4";
  FSVD_REQUIRE_PTR(qweight, fn); FSVD_REQUIRE_PTR(scales, fn); FSVD_REQUIRE_PTR(zeros, fn); FSVD_REQUIRE_PTR(w, fn);
  return launch_dequant_q4(static_cast<const uint8_t*>(qweight), ldq, cu16(scales), static_cast<const int16_t*>(zeros), ldg,
                           group_size, u16(w), ldw, N, K, dtype, static_cast<hipStream_t>(stream));
}

int fsvd_swiglu_linear_q4(const void* p, int64_t ldp, int64_t up_off, const void* gate_q, const void* gate_scales,
                          const void* gate_zeros, const void* up_q, const void* up_scales, const void* up_zeros, int64_t ldq,
                          int64_t ldg, int group_size, void* h, int64_t ldh, int B, int D, int R, int mode, int dtype, void* stream) {
  const char* fn = "fsvd_swiglu_linear_q4";
  FSVD_REQUIRE_PTR(p, fn); FSVD_REQUIRE_PTR(gate_q, fn); FSVD_REQUIRE_PTR(gate_scales, fn); FSVD_REQUIRE_PTR(gate_zeros, fn);
  FSVD_REQUIRE_PTR(up_q, fn); FSVD_REQUIRE_PTR(up_scales, fn); FSVD_REQUIRE_PTR(up_zeros, fn); FSVD_REQUIRE_PTR(h, fn);
  if (up_off < 0 || ldp < up_off + R || ldh < D || (mode != 0 && mode != 1)) {
    set_last_error("%s: inconsistent layout (ldp=%lld up_off=%lld R=%d ldh=%lld D=%d mode=%d)", fn, (long long)ldp,
                   (long long)up_off, R, (long long)ldh, D, mode);
    return kErrBadShape;
  }
  Q4Args a{cu16(p), ldp, up_off, {static_cast<const uint8_t*>(gate_q), static_cast<const uint8_t*>(up_q)}, ldq,
           {cu16(gate_scales), cu16(up_scales)}, {static_cast<const int16_t*>(gate_zeros), static_cast<const int16_t*>(up_zeros)},
           ldg, group_size, nullptr, nullptr, 0.f, nullptr, 0, u16(h), ldh, B, D, R, 2, mode, dtype};
  return launch_linear_q4(a, static_cast<hipStream_t>(stream));
}

int fsvd_qkv_rope_append(const void* p, int64_t ldp, const void* q_u, int64_t ldq, const void* k_u, int64_t ldk,
                         const void* v_u, int64_t ldv, const void* cos, const void* sin, int rope_len,
                         const int32_t* positions, void* q_out, void* k_cache, void* v_cache, int64_t sc_b, int64_t sc_s,
                         int64_t sc_h, int B, int H, int Hk, int Dh, int Rq, int Rk, int Rv, int S, int cfg, int dtype, void* stream) {
  const char* fn = "fsvd_qkv_rope_append";
  FSVD_REQUIRE_PTR(p, fn); FSVD_REQUIRE_PTR(q_u, fn); FSVD_REQUIRE_PTR(k_u, fn); FSVD_REQUIRE_PTR(v_u, fn);
  FSVD_REQUIRE_PTR(positions, fn); FSVD_REQUIRE_PTR(q_out, fn); FSVD_REQUIRE_PTR(k_cache, fn); FSVD_REQUIRE_PTR(v_cache, fn);
  if ((cos == nullptr) != (sin == nullptr) || (cos && rope_len <= 0)) { set_last_error("%s: cos/sin must both be set with rope_len > 0", fn); return kErrBadShape; }
  if (ldp < (int64_t)Rq + Rk + Rv || ldq < Rq || ldk < Rk || ldv < Rv || sc_h < Dh) {
    set_last_error("%s: leading dimensions smaller than the rows", fn);
    return kErrBadShape;
  }
  QkvArgs a{cu16(p), ldp, cu16(q_u), ldq, cu16(k_u), ldk, cu16(v_u), ldv, cu16(cos), cu16(sin), rope_len, positions,
            u16(q_out), u16(k_cache), u16(v_cache), sc_b, sc_s, sc_h, B, H, Hk, Dh, Rq, Rk, Rv, S, dtype};
  return launch_qkv(a, cfg, static_cast<hipStream_t>(stream));
}

// arrival counters (one per (b,h), zero at rest) sit in a fixed-size block at the front of the
// attention workspace, the fp32 partials behind it
static constexpr size_t kAttnCounterBytes = 256 * 1024;

size_t fsvd_attn_decode_workspace_bytes(int B, int H, int Dh, int nsplit) {
  if (B <= 0 || H <= 0 || Dh <= 0 || nsplit <= 0) return 0;
  return kAttnCounterBytes + attn_decode_ws_floats(B, H, nsplit, Dh) * sizeof(float);
}

int fsvd_attn_decode_densekv(const void* q, int64_t sq_b, int64_t sq_h, void* k_cache, void* v_cache, int64_t sc_b,
                             int64_t sc_s, int64_t sc_h, const void* k_new, int64_t sk_b, int64_t sk_h, const void* v_new, int64_t sv_b, int64_t sv_h,
                             const int32_t* cache_seqlens, int seqlen_add, const void* cos, const void* sin, int rope_len,
                             void* out, int64_t so_b, int64_t so_h, void* workspace, size_t workspace_bytes, int B, int H,
                             int Hk, int Dh, int S, int nsplit, float scale, int dtype, void* stream) {
  const char* fn = "fsvd_attn_decode_densekv";
  FSVD_REQUIRE_PTR(q, fn); FSVD_REQUIRE_PTR(k_cache, fn); FSVD_REQUIRE_PTR(v_cache, fn);
  FSVD_REQUIRE_PTR(cache_seqlens, fn); FSVD_REQUIRE_PTR(out, fn);
  if ((cos == nullptr) != (sin == nullptr) || (cos && rope_len <= 0)) { set_last_error("%s: cos/sin must both be set with rope_len > 0", fn); return kErrBadShape; }
  if ((k_new == nullptr) != (v_new == nullptr)) { set_last_error("%s: k_new and v_new must be given together", fn); return kErrNullPtr; }
  if (B <= 0 || H <= 0 || Dh <= 0 || nsplit <= 0) { set_last_error("%s: bad shape", fn); return kErrBadShape; }
  hipStream_t st = static_cast<hipStream_t>(stream);
  float* ws_part = nullptr;
  int32_t* ws_count = nullptr;
  if (nsplit > 1) {
    const size_t need = fsvd_attn_decode_workspace_bytes(B, H, Dh, nsplit);
    if (workspace == nullptr || workspace_bytes < need) {
      set_last_error("%s: workspace of %zu bytes needed, %zu given", fn, need, workspace_bytes);
      return kErrWorkspace;
    }
    if ((size_t)B * H * sizeof(int32_t) > kAttnCounterBytes) {
      set_last_error("%s: B*H = %d exceeds the %zu arrival counters of the workspace", fn, B * H, kAttnCounterBytes / 4);
      return kErrBadShape;
    }
    ws_count = static_cast<int32_t*>(workspace);
    ws_part = reinterpret_cast<float*>(static_cast<char*>(workspace) + kAttnCounterBytes);
  }
  if (k_new) {
    KvAppendArgs ka{cu16(k_new), cu16(v_new), sk_b, sk_h, sv_b, sv_h, u16(k_cache), u16(v_cache), sc_b, sc_s, sc_h,
                    cache_seqlens, cu16(cos), cu16(sin), rope_len, B, Hk, Dh, S, dtype};
    int rc = launch_kv_append(ka, st);
    if (rc != kOk) return rc;
    seqlen_add = 1;
  }
  AttnDecodeArgs a{cu16(q), sq_b, sq_h, cu16(k_cache), cu16(v_cache), sc_b, sc_s, sc_h, cache_seqlens, seqlen_add,
                   cu16(cos), cu16(sin), rope_len, u16(out), so_b, so_h, ws_part, ws_count, B, H, Hk, Dh, S, nsplit,
                   scale > 0.f ? scale : 1.0f / sqrtf((float)Dh), dtype};
  return launch_attn_decode(a, st);
}

// ---- the same attention with library-owned scratch: nothing is allocated and no workspace is passed in -------------
// One array per GPU (each device holds its own copy of a __device__ variable at its own address); its address is
// looked up once per device and only that address, never the array's name, is handed to kernels.
static constexpr size_t kStaticScratchBytes = (size_t)4 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static void* g_static_scratch[kMaxDevices] = {};
static std::mutex g_static_scratch_mu;

static int static_scratch_ptr(void** out, const char* fn) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) { set_last_error("%s: no current device", fn); return kErrLaunch; }
  std::lock_guard<std::mutex> lock(g_static_scratch_mu);
  if (g_static_scratch[dev] == nullptr) {
    void* p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) { set_last_error("%s: hipGetSymbolAddress failed: %s", fn, hipGetErrorString(e)); return kErrLaunch; }
    g_static_scratch[dev] = p;
  }
  *out = g_static_scratch[dev];
  return kOk;
}

size_t fsvd_attn_decode_densekv_static_max_bytes(void) { return kStaticScratchBytes; }

int fsvd_attn_decode_densekv_static(const void* q, int64_t sq_b, int64_t sq_h, void* k_cache, void* v_cache, int64_t sc_b,
                                    int64_t sc_s, int64_t sc_h, const void* k_new, int64_t sk_b, int64_t sk_h, const void* v_new,
                                    int64_t sv_b, int64_t sv_h, const int32_t* cache_seqlens, int seqlen_add, const void* cos,
                                    const void* sin, int rope_len, void* out, int64_t so_b, int64_t so_h, int B, int H, int Hk,
                                    int Dh, int S, int nsplit, float scale, int dtype, void* stream) {
  const char* fn = "fsvd_attn_decode_densekv_static";
  if (B <= 0 || H <= 0 || Dh <= 0 || nsplit <= 0) { set_last_error("%s: bad shape", fn); return kErrBadShape; }
  void* ws = nullptr;
  size_t need = 0;
  if (nsplit > 1) {
    need = fsvd_attn_decode_workspace_bytes(B, H, Dh, nsplit);
    if (need > kStaticScratchBytes) {
      set_last_error("%s: B=%d H=%d Dh=%d nsplit=%d needs %zu bytes of scratch, the built-in array holds %zu "
                     "(use fsvd_attn_decode_densekv with a caller-owned workspace)", fn, B, H, Dh, nsplit, need, kStaticScratchBytes);
      return kErrWorkspace;
    }
    if ((size_t)B * H * sizeof(int32_t) > kAttnCounterBytes) { set_last_error("%s: B*H = %d exceeds the arrival counters", fn, B * H); return kErrBadShape; }
    int rc = static_scratch_ptr(&ws, fn);
    if (rc != kOk) return rc;
    // the array keeps what the previous call left; the arrival counters of this call start at zero whatever that was
    // (a fill kernel, not a memset node: this entry point is meant for callers under stream capture)
    const int ncount = B * H;
    hipLaunchKernelGGL(ws_clear_kernel, dim3((ncount + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<int32_t*>(ws), ncount);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_last_error("%s: launch failed: %s", fn, hipGetErrorString(e)); return kErrLaunch; }
  }
  return fsvd_attn_decode_densekv(q, sq_b, sq_h, k_cache, v_cache, sc_b, sc_s, sc_h, k_new, sk_b, sk_h, v_new, sv_b, sv_h, cache_seqlens,
                                  seqlen_add, cos, sin, rope_len, out, so_b, so_h, ws, need, B, H, Hk, Dh, S, nsplit, scale, dtype, stream);
}

int fsvd_rmsnorm(const void* x, int64_t ldx, const void* w, float eps, void* y, int64_t ldy, int rows, int K, int dtype, void* stream) {
  FSVD_REQUIRE_PTR(x, "fsvd_rmsnorm"); FSVD_REQUIRE_PTR(w, "fsvd_rmsnorm"); FSVD_REQUIRE_PTR(y, "fsvd_rmsnorm");
  return launch_rmsnorm(cu16(x), ldx, cu16(w), eps, u16(y), ldy, rows, K, dtype, static_cast<hipStream_t>(stream));
}

}  // extern "C"

// ---------------------------------------------------------------------------------------------
// reference operand layouts
// ---------------------------------------------------------------------------------------------
namespace {
inline size_t align16(size_t n) { return (n + 15) / 16 * 16; }
inline int esize(int dtype) { return dtype == FSVD_FP32 ? 4 : 2; }

struct XwPlan { XwArgs a; int tx, bt; };

// Workspace layout shared by every split-K entry point: a fixed block of arrival counters at the
// front (zero at rest: each launch leaves its counters at zero) and the fp32 partials behind it.
// The counter block has a fixed size so that calls of different shapes that reuse one workspace
// never see each other's partials as counters.
constexpr size_t kCounterBytes = 64 * 1024;

int run_xw(XwPlan& p, int dtype, char* ws, size_t ws_bytes, const char* fn, hipStream_t st) {
  const size_t pbytes = xw_partial_floats(p.a, p.tx * 8, p.bt) * sizeof(float);
  if (xw_num_tiles(p.a) * sizeof(int32_t) > kCounterBytes) {
    set_last_error("%s: %zu output tiles exceed the %zu arrival counters of the workspace", fn, xw_num_tiles(p.a), kCounterBytes / 4);
    return kErrBadShape;
  }
  if (p.a.ksplit > 1 && (ws == nullptr || ws_bytes < kCounterBytes + pbytes)) {
    set_last_error("%s: workspace of %zu bytes needed, %zu given", fn, kCounterBytes + pbytes, ws_bytes);
    return kErrWorkspace;
  }
  return launch_xw(p.a, dtype, p.tx, p.bt, reinterpret_cast<int32_t*>(ws), reinterpret_cast<float*>(ws + kCounterBytes), st);
}
size_t xw_bytes(const XwPlan& p) {
  return kCounterBytes + xw_partial_floats(p.a, p.tx * 8, p.bt) * sizeof(float);
}

int plan_linear(XwPlan& p, const void* x, int64_t sx_b, int64_t sx_k, int x_fp32, const void* W, int64_t sw_k, const void* bias,
                int bias_post, void* y, int64_t sy_b, int out_fp32, int B, int K, int N, int dtype, int kslice_fixed,
                int round_partials) {
  p.a = XwArgs{};
  p.a.nprob = 1; p.a.B = B; p.a.x_fp32 = x_fp32; p.a.out_fp32 = out_fp32; p.a.round_partials = round_partials; p.a.bias_post = bias_post;
  XwProblem& P = p.a.prob[0];
  P.x = x; P.sx_b = sx_b; P.sx_h = 0; P.sx_k = sx_k; P.W = W; P.sw_h = 0; P.sw_k = sw_k; P.bias = bias; P.sbias_h = 0;
  P.y = y; P.sy_b = sy_b; P.sy_h = 0; P.K = K; P.N = N; P.heads = 1;
  return plan_xw(p.a, dtype, 0, kslice_fixed, &p.tx, &p.bt);
}

int plan_reconstruct(XwPlan& p, const void* const Pm[3], const int64_t sP[3][3], const void* const Vm[3], const int64_t sV[3][2],
                     const void* const bm[3], const int64_t sb[3], void* const Om[3], const int64_t sO[3][2], int B,
                     const int heads[3], int Dh, const int R[3], int dtype) {
  p.a = XwArgs{};
  p.a.nprob = 3; p.a.B = B;
  for (int i = 0; i < 3; ++i) {
    XwProblem& P = p.a.prob[i];
    P.x = Pm[i]; P.sx_b = sP[i][0]; P.sx_h = sP[i][1]; P.sx_k = sP[i][2];
    P.W = Vm[i]; P.sw_h = sV[i][0]; P.sw_k = sV[i][1];
    P.bias = bm[i]; P.sbias_h = sb[i];
    P.y = Om[i]; P.sy_b = sO[i][0]; P.sy_h = sO[i][1];
    P.K = R[i]; P.N = Dh; P.heads = heads[i];
  }
  return plan_xw(p.a, dtype, 0, 0, &p.tx, &p.bt);
}
}  // namespace

extern "C" {

size_t fsvd_xw_linear_workspace_bytes(int B, int K, int N, int dtype) {
  XwPlan p;
  if (plan_linear(p, nullptr, K, 1, 0, nullptr, N, nullptr, 0, nullptr, N, 0, B, K, N, dtype, 0, 0) != kOk) return 0;
  return xw_bytes(p);
}

int fsvd_xw_linear(const void* x, int64_t sx_b, int64_t sx_k, int x_fp32, const void* W, int64_t sw_k, const void* bias,
                   int bias_post, void* y, int64_t sy_b, int out_fp32, int B, int K, int N, int dtype, void* workspace,
                   size_t workspace_bytes, void* stream) {
  const char* fn = "fsvd_xw_linear";
  FSVD_REQUIRE_PTR(x, fn); FSVD_REQUIRE_PTR(W, fn); FSVD_REQUIRE_PTR(y, fn);
  if (dtype < 0 || dtype > 2) { set_last_error("%s: dtype code %d not in {0,1,2}", fn, dtype); return kErrBadDtype; }
  if (sw_k < N || sy_b < N) { set_last_error("%s: leading dimension smaller than N=%d", fn, N); return kErrBadShape; }
  XwPlan p;
  int rc = plan_linear(p, x, sx_b, sx_k, x_fp32, W, sw_k, bias, bias_post, y, sy_b, out_fp32, B, K, N, dtype, 0, 0);
  if (rc != kOk) return rc;
  return run_xw(p, dtype, static_cast<char*>(workspace), workspace_bytes, fn, static_cast<hipStream_t>(stream));
}

size_t fsvd_reconstruct_qkv_workspace_bytes(int B, int H, int Hk, int Dh, int Rq, int Rk, int Rv, int dtype) {
  XwPlan p;
  const void* nul[3] = {nullptr, nullptr, nullptr};
  void* nulo[3] = {nullptr, nullptr, nullptr};
  const int64_t sP[3][3] = {{Rq, 0, 1}, {Rk, 0, 1}, {Rv, 0, 1}};
  const int64_t sV[3][2] = {{(int64_t)Rq * Dh, Dh}, {(int64_t)Rk * Dh, Dh}, {(int64_t)Rv * Dh, Dh}};
  const int64_t sb[3] = {Dh, Dh, Dh};
  const int64_t sO[3][2] = {{(int64_t)H * Dh, Dh}, {(int64_t)Hk * Dh, Dh}, {(int64_t)Hk * Dh, Dh}};
  const int heads[3] = {H, Hk, Hk};
  const int R[3] = {Rq, Rk, Rv};
  if (plan_reconstruct(p, nul, sP, nul, sV, nul, sb, nulo, sO, B, heads, Dh, R, dtype) != kOk) return 0;
  return xw_bytes(p);
}

int fsvd_reconstruct_qkv_token(const void* Pq, int64_t sPq_b, int64_t sPq_h, int64_t sPq_r, const void* Pk, int64_t sPk_b,
                               int64_t sPk_h, int64_t sPk_r, const void* Pv, int64_t sPv_b, int64_t sPv_h, int64_t sPv_r,
                               const void* Vq, int64_t sVq_h, int64_t sVq_r, const void* Vk, int64_t sVk_h, int64_t sVk_r,
                               const void* Vv, int64_t sVv_h, int64_t sVv_r, const void* bq, int64_t sbq_h, const void* bk,
                               int64_t sbk_h, const void* bv, int64_t sbv_h, void* Q, int64_t sQ_b, int64_t sQ_h, void* K,
                               int64_t sK_b, int64_t sK_h, void* V, int64_t sV_b, int64_t sV_h, int B, int H, int Hk, int Dh,
                               int Rq, int Rk, int Rv, int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  const char* fn = "fsvd_reconstruct_qkv_token";
  FSVD_REQUIRE_PTR(Pq, fn); FSVD_REQUIRE_PTR(Pk, fn); FSVD_REQUIRE_PTR(Pv, fn);
  FSVD_REQUIRE_PTR(Vq, fn); FSVD_REQUIRE_PTR(Vk, fn); FSVD_REQUIRE_PTR(Vv, fn);
  FSVD_REQUIRE_PTR(Q, fn); FSVD_REQUIRE_PTR(K, fn); FSVD_REQUIRE_PTR(V, fn);
  if (dtype < 0 || dtype > 2) { set_last_error("%s: dtype code %d not in {0,1,2}", fn, dtype); return kErrBadDtype; }
  if (B <= 0 || H <= 0 || Hk <= 0 || Dh <= 0 || Rq <= 0 || Rk <= 0 || Rv <= 0) {
    set_last_error("%s: bad shape B=%d H=%d Hk=%d Dh=%d R=(%d,%d,%d)", fn, B, H, Hk, Dh, Rq, Rk, Rv);
    return kErrBadShape;
  }
  if (sVq_r < Dh || sVk_r < Dh || sVv_r < Dh || sQ_h < Dh || sK_h < Dh || sV_h < Dh) {
    set_last_error("%s: a row stride is smaller than head_dim %d", fn, Dh);
    return kErrBadShape;
  }
  const void* Pm[3] = {Pq, Pk, Pv};
  const int64_t sP[3][3] = {{sPq_b, sPq_h, sPq_r}, {sPk_b, sPk_h, sPk_r}, {sPv_b, sPv_h, sPv_r}};
  const void* Vm[3] = {Vq, Vk, Vv};
  const int64_t sVm[3][2] = {{sVq_h, sVq_r}, {sVk_h, sVk_r}, {sVv_h, sVv_r}};
  const void* bm[3] = {bq, bk, bv};
  const int64_t sb[3] = {sbq_h, sbk_h, sbv_h};
  void* Om[3] = {Q, K, V};
  const int64_t sO[3][2] = {{sQ_b, sQ_h}, {sK_b, sK_h}, {sV_b, sV_h}};
  const int heads[3] = {H, Hk, Hk};
  const int R[3] = {Rq, Rk, Rv};
  XwPlan p;
  int rc = plan_reconstruct(p, Pm, sP, Vm, sVm, bm, sb, Om, sO, B, heads, Dh, R, dtype);
  if (rc != kOk) return rc;
  return run_xw(p, dtype, static_cast<char*>(workspace), workspace_bytes, fn, static_cast<hipStream_t>(stream));
}

namespace {
struct MlpPlan { XwPlan gu, dv, du; size_t off_h, off_s, off_xw, cbytes, total; };

int plan_mlp(MlpPlan& m, const void* PUp, int64_t sPUp_t, const void* PGate, int64_t sPGate_t, const void* GateU, int64_t ldGateU,
             const void* UpU, int64_t ldUpU, const void* DownV, int64_t ldDownV, const void* DownU, int64_t ldDownU, const void* b2,
             void* Y, int64_t ldY, int T, int R, int D, int Hd, int dtype, int variant, int bd, int partials_fp32, char* ws) {
  const int es = esize(dtype);
  m.off_h = kCounterBytes;
  m.off_s = m.off_h + align16((size_t)T * D * es);
  m.off_xw = m.off_s + align16((size_t)T * R * sizeof(float));
  void* h = ws ? ws + m.off_h : nullptr;
  float* S = ws ? reinterpret_cast<float*>(ws + m.off_s) : nullptr;
  // stage 1: h = silu(PGate @ GateU) * (PUp @ UpU)
  m.gu.a = XwArgs{};
  m.gu.a.nprob = 1; m.gu.a.B = T; m.gu.a.dual = 1;
  XwProblem& G = m.gu.a.prob[0];
  if (ldGateU != ldUpU) { set_last_error("fsvd_mlp_dual_split: GateU and UpU must share a row stride"); return kErrBadShape; }
  G.x = PGate; G.x2 = PUp; G.sx_b = sPGate_t; G.sx_h = 0; G.sx_k = 1; G.W = GateU; G.W2 = UpU; G.sw_h = 0; G.sw_k = ldGateU;
  G.y = h; G.sy_b = D; G.sy_h = 0; G.K = R; G.N = D; G.heads = 1;
  if (sPGate_t != sPUp_t) { set_last_error("fsvd_mlp_dual_split: PUp and PGate must share a row stride"); return kErrBadShape; }
  int rc = plan_xw(m.gu.a, dtype, 0, 0, &m.gu.tx, &m.gu.bt);
  if (rc != kOk) return rc;
  // stage 2: S = h @ DownV, one K slice per D tile of bd rows
  const bool s_fp32 = variant != 1;   // v1 keeps S in dtype (sum of dtype partials); v2/v3 carry fp32
  rc = plan_linear(m.dv, h, D, 1, 0, DownV, ldDownV, nullptr, 0, S, R, s_fp32 ? 1 : 0, T, D, R, dtype, bd,
                   variant == 3 || (variant == 1 && !partials_fp32));
  if (rc != kOk) return rc;
  // stage 3: Y = S @ DownU (+ b2)
  // v1: S already in dtype.  v2: fp32 S rounded to dtype while it is staged.  v3: fp32 S used as is.
  rc = plan_linear(m.du, S, R, 1, s_fp32 ? 1 : 0, DownU, ldDownU, b2, variant == 3 ? 1 : 0, Y, ldY, 0, T, R, Hd, dtype, 0, 0);
  if (rc != kOk) return rc;
  m.du.a.x_round = variant == 2 ? 1 : 0;
  // the three stages run one after another and share the counter block at the front of the
  // workspace and one partials block behind the h and S buffers
  const size_t cbytes = 0;
  if (std::max(xw_num_tiles(m.gu.a), std::max(xw_num_tiles(m.dv.a), xw_num_tiles(m.du.a))) * sizeof(int32_t) > kCounterBytes) {
    set_last_error("fsvd_mlp_dual_split: too many output tiles for the workspace counters");
    return kErrBadShape;
  }
  const size_t pfloats = std::max(xw_partial_floats(m.gu.a, m.gu.tx * 8, m.gu.bt),
                                  std::max(xw_partial_floats(m.dv.a, m.dv.tx * 8, m.dv.bt), xw_partial_floats(m.du.a, m.du.tx * 8, m.du.bt)));
  m.cbytes = cbytes;
  m.total = m.off_xw + cbytes + pfloats * sizeof(float);
  return kOk;
}
}  // namespace

size_t fsvd_mlp_dual_split_workspace_bytes(int T, int R, int D, int Hd, int dtype, int bd) {
  MlpPlan m;
  if (bd <= 0) bd = 128;
  if (plan_mlp(m, nullptr, R, nullptr, R, nullptr, D, nullptr, D, nullptr, R, nullptr, Hd, nullptr, nullptr, Hd, T, R, D, Hd,
               dtype, 2, bd, 1, nullptr) != kOk) return 0;
  return m.total;
}

int fsvd_mlp_dual_split(const void* PUp, int64_t sPUp_t, const void* PGate, int64_t sPGate_t, const void* GateU, int64_t ldGateU,
                        const void* UpU, int64_t ldUpU, const void* DownV, int64_t ldDownV, const void* DownU, int64_t ldDownU,
                        const void* b2, void* Y, int64_t ldY, float* S_out, int T, int R, int D, int Hd, int dtype, int variant,
                        int bd, int partials_fp32, void* workspace, size_t workspace_bytes, void* stream) {
  const char* fn = "fsvd_mlp_dual_split";
  FSVD_REQUIRE_PTR(PUp, fn); FSVD_REQUIRE_PTR(PGate, fn); FSVD_REQUIRE_PTR(GateU, fn); FSVD_REQUIRE_PTR(UpU, fn);
  FSVD_REQUIRE_PTR(DownV, fn); FSVD_REQUIRE_PTR(DownU, fn); FSVD_REQUIRE_PTR(Y, fn); FSVD_REQUIRE_PTR(workspace, fn);
  if (dtype < 0 || dtype > 2) { set_last_error("%s: dtype code %d not in {0,1,2}", fn, dtype); return kErrBadDtype; }
  if (variant < 1 || variant > 3) { set_last_error("%s: variant %d not in {1,2,3}", fn, variant); return kErrBadShape; }
  if (T <= 0 || R <= 0 || D <= 0 || Hd <= 0) { set_last_error("%s: bad shape T=%d R=%d D=%d Hd=%d", fn, T, R, D, Hd); return kErrBadShape; }
  if (ldGateU < D || ldUpU < D || ldDownV < R || ldDownU < Hd || ldY < Hd || sPUp_t < R) {
    set_last_error("%s: a leading dimension is smaller than its row", fn);
    return kErrBadShape;
  }
  if (bd <= 0) bd = 128;
  hipStream_t st = static_cast<hipStream_t>(stream);
  char* ws = static_cast<char*>(workspace);
  MlpPlan m;
  int rc = plan_mlp(m, PUp, sPUp_t, PGate, sPGate_t, GateU, ldGateU, UpU, ldUpU, DownV, ldDownV, DownU, ldDownU, b2, Y, ldY, T, R,
                    D, Hd, dtype, variant, bd, partials_fp32, ws);
  if (rc != kOk) return rc;
  if (workspace_bytes < m.total) { set_last_error("%s: workspace of %zu bytes needed, %zu given", fn, m.total, workspace_bytes); return kErrWorkspace; }
  int32_t* counters = reinterpret_cast<int32_t*>(ws);
  float* partials = reinterpret_cast<float*>(ws + m.off_xw);
  rc = launch_xw(m.gu.a, dtype, m.gu.tx, m.gu.bt, counters, partials, st);
  if (rc != kOk) return rc;
  rc = launch_xw(m.dv.a, dtype, m.dv.tx, m.dv.bt, counters, partials, st);
  if (rc != kOk) return rc;
  if (variant != 1 && S_out) {
    hipError_t e = hipMemcpyAsync(S_out, ws + m.off_s, (size_t)T * R * sizeof(float), hipMemcpyDeviceToDevice, st);
    if (e != hipSuccess) { set_last_error("%s: copy of S failed: %s", fn, hipGetErrorString(e)); return kErrLaunch; }
  }
  return launch_xw(m.du.a, dtype, m.du.tx, m.du.bt, counters, partials, st);
}

size_t fsvd_attn_decode_rankkv_scores_bytes(int B, int H, int S, int shared_by_heads) {
  return rank_decode_scores_floats(B, H, S, shared_by_heads ? 0 : 1) * sizeof(float);
}

int fsvd_attn_decode_rankkv(const void* q, int64_t sq_b, int64_t sq_h, const void* pk_cache, int64_t spk_b, int64_t spk_s, int64_t spk_h,
                            const void* pv_cache, int64_t spv_b, int64_t spv_s, int64_t spv_h, const void* k_u, int64_t ldku, const void* v_u,
                            int64_t ldvu, const void* bv, const void* cos, const void* sin, int rope_len, int rotate_q,
                            const int32_t* cache_seqlens, int seqlen_add, float* ws_m, float* ws_l, float* ws_acc, void* out,
                            int64_t so_b, int64_t so_h, int B, int H, int Hk, int Dh, int S, int Rk, int Rv, int nsplit,
                            float scale, float* scores, size_t scores_bytes, int dtype, void* stream) {
  const char* fn = "fsvd_attn_decode_rankkv";
  FSVD_REQUIRE_PTR(q, fn); FSVD_REQUIRE_PTR(pk_cache, fn); FSVD_REQUIRE_PTR(pv_cache, fn); FSVD_REQUIRE_PTR(k_u, fn);
  FSVD_REQUIRE_PTR(v_u, fn); FSVD_REQUIRE_PTR(cache_seqlens, fn); FSVD_REQUIRE_PTR(ws_m, fn); FSVD_REQUIRE_PTR(ws_l, fn);
  FSVD_REQUIRE_PTR(ws_acc, fn); FSVD_REQUIRE_PTR(out, fn);
  if ((cos == nullptr) != (sin == nullptr) || (cos && rope_len <= 0)) { set_last_error("%s: cos/sin must both be set with rope_len > 0", fn); return kErrBadShape; }
  if (rotate_q && !cos) { set_last_error("%s: rotate_q needs cos/sin tables", fn); return kErrBadShape; }
  if (spk_s < Rk || spv_s < Rv || ldku < Rk || ldvu < Rv) { set_last_error("%s: a row stride is smaller than its rank", fn); return kErrBadShape; }
  RankDecodeArgs a{cu16(q), sq_b, sq_h, cu16(pk_cache), spk_b, spk_s, spk_h, cu16(pv_cache), spv_b, spv_s, spv_h, cu16(k_u), ldku, cu16(v_u), ldvu,
                   cu16(bv), cu16(cos), cu16(sin), rope_len, rotate_q, cache_seqlens, seqlen_add, ws_m, ws_l, ws_acc, u16(out),
                   so_b, so_h, B, H, Hk, Dh, S, Rk, Rv, nsplit, scale > 0.f ? scale : 1.0f / sqrtf((float)Dh)};
  if (scores != nullptr) {
    const size_t need = rank_decode_scores_floats(B, H, S, spv_h) * sizeof(float);
    if (need != 0 && scores_bytes < need) {
      set_last_error("%s: the score buffer holds %zu bytes, this shape needs %zu (fsvd_attn_decode_rankkv_scores_bytes)", fn, scores_bytes, need);
      return kErrWorkspace;
    }
    if ((reinterpret_cast<uintptr_t>(scores) & 15) != 0) { set_last_error("%s: the score buffer must be 16-byte aligned", fn); return kErrBadAlign; }
    a.scores = scores;
  }
  a.dt = dtype;
  return launch_rank_decode(a, static_cast<hipStream_t>(stream));
}

int fsvd_rankkv_append(const void* pk, int64_t ldpk, const void* pv, int64_t ldpv, void* pk_cache, int64_t spk_b, int64_t spk_s,
                       void* pv_cache, int64_t spv_b, int64_t spv_s, const int32_t* positions, int B, int S, int Rk, int Rv, void* stream) {
  const char* fn = "fsvd_rankkv_append";
  FSVD_REQUIRE_PTR(pk, fn); FSVD_REQUIRE_PTR(pv, fn); FSVD_REQUIRE_PTR(pk_cache, fn); FSVD_REQUIRE_PTR(pv_cache, fn); FSVD_REQUIRE_PTR(positions, fn);
  if (B <= 0 || S <= 0 || Rk <= 0 || Rv <= 0 || (Rk % 8) || (Rv % 8) || ldpk < Rk || ldpv < Rv || spk_s < Rk || spv_s < Rv) {
    set_last_error("%s: bad shape B=%d S=%d Rk=%d Rv=%d (ranks are multiples of 8, row strides at least the rank)", fn, B, S, Rk, Rv);
    return kErrBadShape;
  }
  const auto mis = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) != 0; };
  if (mis(pk) || mis(pv) || mis(pk_cache) || mis(pv_cache) || (ldpk % 8) || (ldpv % 8) || (spk_b % 8) || (spk_s % 8) || (spv_b % 8) || (spv_s % 8)) {
    set_last_error("%s: pointers and strides must be 16-byte aligned", fn);
    return kErrBadAlign;
  }
  return launch_rankkv_append(cu16(pk), ldpk, cu16(pv), ldpv, u16(pk_cache), spk_b, spk_s, u16(pv_cache), spv_b, spv_s, positions, B, S, Rk, Rv,
                              static_cast<hipStream_t>(stream));
}

int fsvd_lowrank_expand_heads(const void* p, int64_t sp_b, int64_t sp_m, int64_t sp_h, const void* u, int64_t ldu, const void* bias,
                              const void* cos, const void* sin, int rope_len, const int32_t* positions, void* y, int64_t sy_b,
                              int64_t sy_m, int64_t sy_h, int dst_by_position, int dst_rows, int B, int M, int heads, int Dh, int R,
                              int dtype, void* stream) {
  const char* fn = "fsvd_lowrank_expand_heads";
  FSVD_REQUIRE_PTR(p, fn); FSVD_REQUIRE_PTR(u, fn); FSVD_REQUIRE_PTR(y, fn);
  if ((cos == nullptr) != (sin == nullptr) || (cos && rope_len <= 0)) { set_last_error("%s: cos/sin must both be set with rope_len > 0", fn); return kErrBadShape; }
  if (ldu < R || sy_h < Dh || dst_rows <= 0) { set_last_error("%s: inconsistent strides (ldu=%lld R=%d sy_h=%lld dst_rows=%d)", fn, (long long)ldu, R, (long long)sy_h, dst_rows); return kErrBadShape; }
  ExpandArgs a{cu16(p), sp_b, sp_m, sp_h, cu16(u), ldu, cu16(bias), cu16(cos), cu16(sin), rope_len, positions, u16(y), sy_b, sy_m,
               sy_h, dst_by_position, dst_rows, B, M, heads, Dh, R, dtype};
  return launch_expand(a, static_cast<hipStream_t>(stream));
}

int fsvd_lowrank_expand_heads_multi(const fsvd_expand_desc* desc, int n, const void* cos, const void* sin, int rope_len,
                                    const int32_t* positions, int B, int M, int Dh, int dtype, void* stream) {
  const char* fn = "fsvd_lowrank_expand_heads_multi";
  FSVD_REQUIRE_PTR(desc, fn);
  if (n < 1 || n > 3) { set_last_error("%s: %d descriptors (1..3)", fn, n); return kErrBadShape; }
  if ((cos == nullptr) != (sin == nullptr) || (cos && rope_len <= 0)) { set_last_error("%s: cos/sin must both be set with rope_len > 0", fn); return kErrBadShape; }
  ExpandArgs a[3];
  for (int k = 0; k < n; ++k) {
    const fsvd_expand_desc& d = desc[k];
    FSVD_REQUIRE_PTR(d.p, fn); FSVD_REQUIRE_PTR(d.u, fn); FSVD_REQUIRE_PTR(d.y, fn);
    if (d.rotate && !cos) { set_last_error("%s: descriptor %d asks for the rotation but no tables were given", fn, k); return kErrBadShape; }
    if (d.ldu < d.R || d.sy_h < Dh || d.dst_rows <= 0) {
      set_last_error("%s: descriptor %d: inconsistent strides (ldu=%lld R=%d sy_h=%lld dst_rows=%d)", fn, k, (long long)d.ldu, d.R, (long long)d.sy_h, d.dst_rows);
      return kErrBadShape;
    }
    a[k] = ExpandArgs{cu16(d.p), d.sp_b, d.sp_m, d.sp_h, cu16(d.u), d.ldu, cu16(d.bias), d.rotate ? cu16(cos) : nullptr,
                      d.rotate ? cu16(sin) : nullptr, rope_len, positions, u16(d.y), d.sy_b, d.sy_m, d.sy_h, d.dst_by_position,
                      d.dst_rows, B, M, d.heads, Dh, d.R, dtype};
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (expand_multi_apply(a, n)) {
    // the single-expansion checks (head_dim, alignment) hold for every descriptor: expand_tiles_apply covers strides
    // and rank, the pointers are checked here
    bool ok = true;
    for (int k = 0; k < n; ++k) ok = ok && ((reinterpret_cast<uintptr_t>(a[k].p) | reinterpret_cast<uintptr_t>(a[k].u)) & 15) == 0 && (a[k].sp_h % 8) == 0;
    if (ok) return launch_expand_multi(a, n, st);
  }
  for (int k = 0; k < n; ++k) {
    const int rc = launch_expand(a[k], st);
    if (rc != kOk) return rc;
  }
  return kOk;
}

int fsvd_attn_prefill(const void* q, int64_t sq_b, int64_t sq_m, int64_t sq_h, const void* k, const void* v, int64_t sk_b,
                      int64_t sk_s, int64_t sk_h, const int32_t* q_pos0, const uint8_t* pad_mask, int64_t spm_b,
                      const float* add_mask, int64_t sam_b, int64_t sam_q, void* out, int64_t so_b, int64_t so_m, int64_t so_h,
                      int B, int M, int H, int Hk, int Dh, int S, int causal, float scale, int dtype, void* stream) {
  const char* fn = "fsvd_attn_prefill";
  FSVD_REQUIRE_PTR(q, fn); FSVD_REQUIRE_PTR(k, fn); FSVD_REQUIRE_PTR(v, fn); FSVD_REQUIRE_PTR(out, fn);
  if (S <= 0 || (!q_pos0 && M > S)) { set_last_error("%s: %d queries do not fit %d cache rows", fn, M, S); return kErrBadShape; }
  PrefillAttnArgs a{cu16(q), sq_b, sq_m, sq_h, cu16(k), cu16(v), sk_b, sk_s, sk_h, q_pos0, pad_mask, spm_b, add_mask, sam_b, sam_q,
                    u16(out), so_b, so_m, so_h, B, M, H, Hk, Dh, S, causal, scale > 0.f ? scale : 1.0f / sqrtf((float)Dh), dtype};
  return launch_prefill_attn(a, static_cast<hipStream_t>(stream));
}

int fsvd_decode_step_workgroups(void) { return decode_step_workgroups(); }

int fsvd_decode_step_prepare(fsvd_phase* phases_host, int nphase, int workgroups) {
  const char* fn = "fsvd_decode_step_prepare";
  FSVD_REQUIRE_PTR(phases_host, fn);
  if (nphase <= 0 || workgroups <= 0) { set_last_error("%s: bad arguments", fn); return kErrBadShape; }
  return prepare_decode_step(phases_host, nphase, workgroups);
}

int fsvd_decode_step_validate(const fsvd_phase* phases_host, int nphase, int workgroups) {
  const char* fn = "fsvd_decode_step_validate";
  FSVD_REQUIRE_PTR(phases_host, fn);
  if (nphase <= 0 || workgroups <= 0) { set_last_error("%s: bad arguments", fn); return kErrBadShape; }
  return validate_decode_step(phases_host, nphase, workgroups);
}

int fsvd_decode_step(const fsvd_phase* phases_dev, const fsvd_phase* phases_host, int nphase, fsvd_step_state* state,
                     int validate, void* stream) {
  const char* fn = "fsvd_decode_step";
  FSVD_REQUIRE_PTR(phases_dev, fn); FSVD_REQUIRE_PTR(state, fn);
  if (nphase <= 0) { set_last_error("%s: empty phase list", fn); return kErrBadShape; }
  if (validate) {
    FSVD_REQUIRE_PTR(phases_host, fn);
    const int nwg = decode_step_workgroups();
    if (nwg <= 0) return kErrLaunch;   // decode_step_workgroups left the reason in the last-error text
    const int rc = validate_decode_step(phases_host, nphase, nwg);
    if (rc != kOk) return rc;
  }
  return launch_decode_step(phases_dev, nphase, state, nullptr, 1, decode_step_build(phases_host, nphase), static_cast<hipStream_t>(stream));
}

int fsvd_decode_step_trace(const fsvd_phase* phases_dev, const fsvd_phase* phases_host, int nphase, fsvd_step_state* state,
                           uint64_t* trace, size_t trace_words, int wg_stride, void* stream) {
  const char* fn = "fsvd_decode_step_trace";
  FSVD_REQUIRE_PTR(phases_dev, fn); FSVD_REQUIRE_PTR(state, fn); FSVD_REQUIRE_PTR(trace, fn);
  const int nwg = decode_step_workgroups();
  if (nwg <= 0) return kErrLaunch;
  if (nphase <= 0 || wg_stride <= 0) { set_last_error("%s: bad arguments", fn); return kErrBadShape; }
  const size_t need = (size_t)((nwg + wg_stride - 1) / wg_stride) * nphase * 4;
  if (trace_words < need) { set_last_error("%s: trace buffer holds %zu words, %zu needed", fn, trace_words, need); return kErrWorkspace; }
  return launch_decode_step(phases_dev, nphase, state, reinterpret_cast<unsigned long long*>(trace), wg_stride,
                            decode_step_build(phases_host, nphase), static_cast<hipStream_t>(stream));
}

}  // extern "C"
