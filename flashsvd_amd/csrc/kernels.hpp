// Argument blocks and host launchers shared between the kernel files and the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fsvd {

struct LinearArgs {
  const uint16_t* x; int64_t ldx;        // [B, K] activations (bf16)
  const uint16_t* W; int64_t ldw;        // [N, K] nn.Linear weight
  const uint16_t* bias;                  // [N] or null
  const uint16_t* norm_w; float eps;     // fused RMSNorm over x when non-null
  const uint16_t* res; int64_t ldres;    // residual [B, N] or null
  uint16_t* y; int64_t ldy;              // [B, N]
  int B, N, K;
};

struct SwigluArgs {
  const uint16_t* p; int64_t ldp; int64_t up_off;  // [B, >=up_off+R]: gate input at 0, up input at up_off
  const uint16_t* gate_u; const uint16_t* up_u; int64_t ldw;  // [D, R] each
  uint16_t* h; int64_t ldh;              // [B, D]
  int B, D, R;
  int mode;                              // 0 chain-of-linears rounding, 1 fused-kernel rounding
};

struct QkvArgs {
  const uint16_t* p; int64_t ldp;        // [B, Rq+Rk+Rv] packed rank coefficients
  const uint16_t* q_u; int64_t ldq;      // [H*Dh, Rq]
  const uint16_t* k_u; int64_t ldk;      // [Hk*Dh, Rk]
  const uint16_t* v_u; int64_t ldv;      // [Hk*Dh, Rv]
  const uint16_t* cos; const uint16_t* sin; int rope_len;  // [rope_len, Dh/2] or null
  const int32_t* positions;              // [B] write position / rotary position
  uint16_t* q_out;                       // [B, H, Dh]
  uint16_t* k_cache; uint16_t* v_cache;  // [B, S, Hk, Dh] with element strides below
  int64_t sc_b, sc_s, sc_h;
  int B, H, Hk, Dh, Rq, Rk, Rv, S;
};

struct AttnDecodeArgs {
  const uint16_t* q;                     // [B, H, Dh] (sq_b, sq_h strides)
  int64_t sq_b, sq_h;
  const uint16_t* k_cache; const uint16_t* v_cache;  // [B, S, Hk, Dh]
  int64_t sc_b, sc_s, sc_h;
  const int32_t* seqlens;                // [B] number of valid keys
  int seqlen_add;                        // added to seqlens[b] (1 when the new token was just appended)
  const uint16_t* cos; const uint16_t* sin; int rope_len;  // optional in-kernel rotation of q at position seqlens[b]
  uint16_t* out; int64_t so_b, so_h;     // [B, H, Dh]
  float* ws_part;                        // [B, H, nsplit, Dh + 2] fp32 partials
  int32_t* ws_count;                     // [B, H] arrival counters (zero before first use; self-resetting)
  int B, H, Hk, Dh, S, nsplit;
  float scale;
};

struct KvAppendArgs {
  const uint16_t* k_new; const uint16_t* v_new;  // [B, Hk, Dh]
  int64_t sk_b, sk_h, sv_b, sv_h;
  uint16_t* k_cache; uint16_t* v_cache; int64_t sc_b, sc_s, sc_h;
  const int32_t* seqlens;
  const uint16_t* cos; const uint16_t* sin; int rope_len;
  int B, Hk, Dh, S;
};

int launch_linear(const LinearArgs& a, int cfg, hipStream_t st);
int launch_swiglu(const SwigluArgs& a, int cfg, hipStream_t st);
int launch_qkv(const QkvArgs& a, int cfg, hipStream_t st);
int launch_rmsnorm(const uint16_t* x, int64_t ldx, const uint16_t* w, float eps, uint16_t* y, int64_t ldy, int rows,
                   int K, hipStream_t st);
int launch_attn_decode(const AttnDecodeArgs& a, hipStream_t st);
int launch_kv_append(const KvAppendArgs& a, hipStream_t st);
size_t attn_decode_ws_floats(int B, int H, int nsplit, int Dh);

}  // namespace fsvd
