// extern "C" surface of libflashsvd_hip: argument checks, then the launchers.
#include <cstdarg>
#include <cstdio>
#include <cstring>

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

using namespace fsvd;

#define FSVD_REQUIRE_PTR(p, fn)                             \
  if ((p) == nullptr) {                                     \
    set_last_error("%s: argument %s is NULL", fn, #p);      \
    return kErrNullPtr;                                     \
  }

static inline const uint16_t* cu16(const void* p) { return static_cast<const uint16_t*>(p); }
static inline uint16_t* u16(void* p) { return static_cast<uint16_t*>(p); }

extern "C" {

int fsvd_version(void) { return 100; }
const char* fsvd_last_error(void) { return g_last_error; }

int fsvd_linear(const void* x, int64_t ldx, const void* W, int64_t ldw, const void* bias, const void* norm_w, float eps,
                const void* res, int64_t ldres, void* y, int64_t ldy, int B, int N, int K, int cfg, void* stream) {
  FSVD_REQUIRE_PTR(x, "fsvd_linear"); FSVD_REQUIRE_PTR(W, "fsvd_linear"); FSVD_REQUIRE_PTR(y, "fsvd_linear");
  if (ldx < K || ldw < K || ldy < N || (res && ldres < N)) {
    set_last_error("fsvd_linear: leading dimension smaller than the row (ldx=%lld ldw=%lld ldy=%lld ldres=%lld K=%d N=%d)",
                   (long long)ldx, (long long)ldw, (long long)ldy, (long long)ldres, K, N);
    return kErrBadShape;
  }
  LinearArgs a{cu16(x), ldx, cu16(W), ldw, cu16(bias), cu16(norm_w), eps, cu16(res), ldres, u16(y), ldy, B, N, K};
  return launch_linear(a, cfg, static_cast<hipStream_t>(stream));
}

int fsvd_swiglu_linear(const void* p, int64_t ldp, int64_t up_off, const void* gate_u, const void* up_u, int64_t ldw,
                       void* h, int64_t ldh, int B, int D, int R, int mode, int cfg, void* stream) {
  FSVD_REQUIRE_PTR(p, "fsvd_swiglu_linear"); FSVD_REQUIRE_PTR(gate_u, "fsvd_swiglu_linear");
  FSVD_REQUIRE_PTR(up_u, "fsvd_swiglu_linear"); FSVD_REQUIRE_PTR(h, "fsvd_swiglu_linear");
  if (up_off < 0 || ldp < up_off + R || ldw < R || ldh < D || (mode != 0 && mode != 1)) {
    set_last_error("fsvd_swiglu_linear: inconsistent layout (ldp=%lld up_off=%lld R=%d ldw=%lld ldh=%lld D=%d mode=%d)",
                   (long long)ldp, (long long)up_off, R, (long long)ldw, (long long)ldh, D, mode);
    return kErrBadShape;
  }
  SwigluArgs a{cu16(p), ldp, up_off, cu16(gate_u), cu16(up_u), ldw, u16(h), ldh, B, D, R, mode};
  return launch_swiglu(a, cfg, static_cast<hipStream_t>(stream));
}

int fsvd_qkv_rope_append(const void* p, int64_t ldp, const void* q_u, int64_t ldq, const void* k_u, int64_t ldk,
                         const void* v_u, int64_t ldv, const void* cos, const void* sin, int rope_len,
                         const int32_t* positions, void* q_out, void* k_cache, void* v_cache, int64_t sc_b, int64_t sc_s,
                         int64_t sc_h, int B, int H, int Hk, int Dh, int Rq, int Rk, int Rv, int S, int cfg, void* stream) {
  const char* fn = "fsvd_qkv_rope_append";
  FSVD_REQUIRE_PTR(p, fn); FSVD_REQUIRE_PTR(q_u, fn); FSVD_REQUIRE_PTR(k_u, fn); FSVD_REQUIRE_PTR(v_u, fn);
  FSVD_REQUIRE_PTR(positions, fn); FSVD_REQUIRE_PTR(q_out, fn); FSVD_REQUIRE_PTR(k_cache, fn); FSVD_REQUIRE_PTR(v_cache, fn);
  if ((cos == nullptr) != (sin == nullptr) || (cos && rope_len <= 0)) { set_last_error("%s: cos/sin must both be set with rope_len > 0", fn); return kErrBadShape; }
  if (ldp < (int64_t)Rq + Rk + Rv || ldq < Rq || ldk < Rk || ldv < Rv || sc_h < Dh) {
    set_last_error("%s: leading dimensions smaller than the rows", fn);
    return kErrBadShape;
  }
  QkvArgs a{cu16(p), ldp, cu16(q_u), ldq, cu16(k_u), ldk, cu16(v_u), ldv, cu16(cos), cu16(sin), rope_len, positions,
            u16(q_out), u16(k_cache), u16(v_cache), sc_b, sc_s, sc_h, B, H, Hk, Dh, Rq, Rk, Rv, S};
  return launch_qkv(a, cfg, static_cast<hipStream_t>(stream));
}

size_t fsvd_attn_decode_workspace_bytes(int B, int H, int Dh, int nsplit) {
  if (B <= 0 || H <= 0 || Dh <= 0 || nsplit <= 0) return 0;
  return attn_decode_ws_floats(B, H, nsplit, Dh) * sizeof(float) + (size_t)B * H * sizeof(int32_t);
}

int fsvd_attn_decode_densekv(const void* q, int64_t sq_b, int64_t sq_h, void* k_cache, void* v_cache, int64_t sc_b,
                             int64_t sc_s, int64_t sc_h, const void* k_new, int64_t sk_b, int64_t sk_h, const void* v_new, int64_t sv_b, int64_t sv_h,
                             const int32_t* cache_seqlens, int seqlen_add, const void* cos, const void* sin, int rope_len,
                             void* out, int64_t so_b, int64_t so_h, void* workspace, size_t workspace_bytes, int B, int H,
                             int Hk, int Dh, int S, int nsplit, float scale, void* stream) {
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
    ws_part = static_cast<float*>(workspace);
    ws_count = reinterpret_cast<int32_t*>(ws_part + attn_decode_ws_floats(B, H, nsplit, Dh));
  }
  if (k_new) {
    KvAppendArgs ka{cu16(k_new), cu16(v_new), sk_b, sk_h, sv_b, sv_h, u16(k_cache), u16(v_cache), sc_b, sc_s, sc_h,
                    cache_seqlens, cu16(cos), cu16(sin), rope_len, B, Hk, Dh, S};
    int rc = launch_kv_append(ka, st);
    if (rc != kOk) return rc;
    seqlen_add = 1;
  }
  AttnDecodeArgs a{cu16(q), sq_b, sq_h, cu16(k_cache), cu16(v_cache), sc_b, sc_s, sc_h, cache_seqlens, seqlen_add,
                   cu16(cos), cu16(sin), rope_len, u16(out), so_b, so_h, ws_part, ws_count, B, H, Hk, Dh, S, nsplit,
                   scale > 0.f ? scale : 1.0f / sqrtf((float)Dh)};
  return launch_attn_decode(a, st);
}

int fsvd_rmsnorm(const void* x, int64_t ldx, const void* w, float eps, void* y, int64_t ldy, int rows, int K, void* stream) {
  FSVD_REQUIRE_PTR(x, "fsvd_rmsnorm"); FSVD_REQUIRE_PTR(w, "fsvd_rmsnorm"); FSVD_REQUIRE_PTR(y, "fsvd_rmsnorm");
  return launch_rmsnorm(cu16(x), ldx, cu16(w), eps, u16(y), ldy, rows, K, static_cast<hipStream_t>(stream));
}

}  // extern "C"
