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
  int dt = 0;                            // element type: 0 bf16, 1 fp16
  // optional second destination of two column ranges of y (one decoded token's coefficients into a rank-space cache):
  // y[b, app_n0[i] + j], j < app_n[i], is also stored at app[i][b * app_sb[i] + positions[b] * app_ss[i] + j] when
  // positions[b] lies in [0, app_S).  Served by the one- and two-row kernels only.
  const int32_t* positions = nullptr;
  uint16_t* app[2] = {nullptr, nullptr};
  int64_t app_sb[2] = {0, 0}, app_ss[2] = {0, 0};
  int app_n0[2] = {0, 0}, app_n[2] = {0, 0};
  int app_S = 0;
};

struct SwigluArgs {
  const uint16_t* p; int64_t ldp; int64_t up_off;  // [B, >=up_off+R]: gate input at 0, up input at up_off
  const uint16_t* gate_u; const uint16_t* up_u; int64_t ldw;  // [D, R] each
  uint16_t* h; int64_t ldh;              // [B, D]
  int B, D, R;
  int mode;                              // 0 chain-of-linears rounding, 1 fused-kernel rounding
  int dt = 0;
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
  int dt = 0;
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
  int dt = 0;
};

struct KvAppendArgs {
  const uint16_t* k_new; const uint16_t* v_new;  // [B, Hk, Dh]
  int64_t sk_b, sk_h, sv_b, sv_h;
  uint16_t* k_cache; uint16_t* v_cache; int64_t sc_b, sc_s, sc_h;
  const int32_t* seqlens;
  const uint16_t* cos; const uint16_t* sin; int rope_len;
  int B, Hk, Dh, S;
  int dt = 0;
};

// one x @ W problem of the input-major GEMV (a launch carries up to three: q, k, v)
struct XwProblem {
  const void* x; const void* x2;         // [B, (heads), K]; x2 feeds W2 in dual mode
  int64_t sx_b, sx_h, sx_k;
  const void* W; const void* W2;         // [(heads), K, N], unit stride along N
  int64_t sw_h, sw_k;
  const void* bias; int64_t sbias_h;     // [(heads), N] or null
  void* y; int64_t sy_b, sy_h;           // [B, (heads), N]
  int K, N, heads;
  int kslice;                            // filled by plan_xw
  int vec;                               // filled by plan_xw: 16-byte loads are legal
};

struct XwArgs {
  XwProblem prob[3];
  int nprob;
  int B;
  int dual;            // 1: y = silu(x@W) * (x2@W2)
  int x_fp32;          // activations are fp32 even though W is 16-bit
  int x_round;         // round the staged activations to the element type (fp32 S -> dtype S)
  int out_fp32;        // store y as fp32
  int round_partials;  // round each K-slice partial to the element type before the final sum
  int bias_post;       // y = round(round(x@W) + bias) instead of round(x@W + bias)
  int ksplit, ntiles_n, grid_x, grid_z;   // filled by plan_xw
  float* ws; int32_t* counters;           // filled by launch_xw
};

int plan_xw(XwArgs& a, int dtype, int want_ksplit, int kslice_fixed, int* tx_out, int* batch_tile_out);
size_t xw_num_tiles(const XwArgs& a);
size_t xw_partial_floats(const XwArgs& a, int tn, int batch_tile);
int launch_xw(XwArgs& a, int dtype, int tx, int batch_tile, int32_t* counters, float* partials, hipStream_t st);

struct RankDecodeArgs {
  const uint16_t* q; int64_t sq_b, sq_h;            // [B,H,Dh] current-token query (bf16)
  const uint16_t* pk; int64_t spk_b, spk_s, spk_h;  // rank-space key cache   [B,S,(Hk),Rk]; head stride 0 when shared
  const uint16_t* pv; int64_t spv_b, spv_s, spv_h;  // rank-space value cache [B,S,(Hk),Rv]
  const uint16_t* k_u; int64_t ldku;                // [Hk*Dh, Rk] nn.Linear layout
  const uint16_t* v_u; int64_t ldvu;                // [Hk*Dh, Rv]
  const uint16_t* bv;                               // [Hk*Dh] or null
  const uint16_t* cos; const uint16_t* sin; int rope_len;   // [rope_len, Dh/2] or null (no rotation of K)
  int rotate_q;                                     // also rotate q at position n_keys-1
  const int32_t* seqlens; int seqlen_add;
  float* ws_m; float* ws_l; float* ws_acc;          // [B,H,nsplit], [B,H,nsplit], [B,H,nsplit,Rv]
  uint16_t* out; int64_t so_b, so_h;                // [B,H,Dh]
  int B, H, Hk, Dh, S, Rk, Rv, nsplit;
  float scale;
  float* scores = nullptr; int64_t score_ld = 0;    // the caller's score buffer [B,H,ceil64(S)] fp32 or null; score_ld is set by the launcher
  int dt = 0;                                       // element type: 0 bf16, 1 fp16
  int split_major = 0;                              // set by the launcher: the splits of a head are neighbours (else the heads of a split)
};
size_t rank_decode_scores_floats(int B, int H, int S, int64_t spv_h);
int launch_rank_decode(const RankDecodeArgs& a, hipStream_t st);
int launch_rankkv_append(const uint16_t* pk, int64_t ldpk, const uint16_t* pv, int64_t ldpv, uint16_t* pkc, int64_t spk_b, int64_t spk_s,
                         uint16_t* pvc, int64_t spv_b, int64_t spv_s, const int32_t* positions, int B, int S, int Rk, int Rv, hipStream_t st);

struct ExpandArgs {
  const uint16_t* p; int64_t sp_b, sp_m, sp_h;      // rank coefficients [B,M,(heads),R]; sp_h = 0 when shared
  const uint16_t* u; int64_t ldu;                   // [heads*Dh, R] nn.Linear layout
  const uint16_t* bias;                             // [heads*Dh] or null
  const uint16_t* cos; const uint16_t* sin; int rope_len;   // rotation tables or null
  const int32_t* positions;                         // [B] absolute position of token 0 of each row (null = 0)
  uint16_t* y; int64_t sy_b, sy_m, sy_h;            // destination [B, rows, heads, Dh]
  int dst_by_position;                              // 1: destination row = absolute position (cache), 0: row = m
  int dst_rows;                                     // rows the destination has (bounds check)
  int B, M, heads, Dh, R;
  int dt = 0;
};
struct PrefillAttnArgs {
  const uint16_t* q; int64_t sq_b, sq_m, sq_h;      // [B,M,H,Dh], rotated
  const uint16_t* k; const uint16_t* v; int64_t sk_b, sk_s, sk_h;   // [B,S,Hk,Dh]
  const int32_t* q_pos0;                            // [B] absolute position of query row 0 (null = 0)
  const uint8_t* pad_mask; int64_t spm_b;           // [B, keys] 1 = valid, or null
  const float* add_mask; int64_t sam_b, sam_q;      // [B, M, keys] additive, or null
  uint16_t* out; int64_t so_b, so_m, so_h;          // [B,M,H,Dh]
  int B, M, H, Hk, Dh, S, causal;
  float scale;
  int dt = 0;
};
int launch_expand(const ExpandArgs& a, hipStream_t st);
bool expand_tiles_apply(const ExpandArgs& a);                               // mfma_gemm.hip
int launch_expand_tiles(const ExpandArgs& a, hipStream_t st);
bool expand_multi_apply(const ExpandArgs* d, int n);                        // two or three expansions in one launch
int launch_expand_multi(const ExpandArgs* d, int n, hipStream_t st);
int launch_prefill_attn(const PrefillAttnArgs& a, hipStream_t st);

// matrix-core projections: y = epilogue(x . W^T) with the rounding points of the vector kernels
struct MfmaArgs {
  const uint16_t* x; int64_t ldx;            // [B, >= K] activations; DUAL: gate input at 0, up input at up_off
  int64_t up_off;
  const uint16_t* W; const uint16_t* W2; int64_t ldw;   // [N, K] (DUAL: gate_u, up_u)
  const uint16_t* bias; const uint16_t* res; int64_t ldres;
  uint16_t* y; int64_t ldy;
  int B, N, K, mode;
  // K split over gridDim.z workgroups per output tile (filled by the launcher when a workspace is registered):
  // fp32 partial tiles and one arrival counter per tile; the last workgroup to arrive adds the partials in order
  int ksplit; float* ws_part; int32_t* ws_count;
  int dt = 0;
};
// caller-owned scratch of the current device for the K-split projections (null when none is registered)
struct SplitWorkspace { float* part; size_t part_floats; int32_t* count; int ncount; };
SplitWorkspace split_workspace();                                            // capi.hip
bool gemm_tiles_apply(const MfmaArgs& a);                                   // mfma_gemm.hip: 128 rows and more
int launch_gemm_tiles(const MfmaArgs& a, bool dual, hipStream_t st, const char* who);
bool gemm_rows_apply(const MfmaArgs& a);                                    // mfma_gemm.hip: 5..127 rows, K split
int launch_gemm_rows(const MfmaArgs& a, bool dual, hipStream_t st, const char* who);

int launch_linear(const LinearArgs& a, int cfg, hipStream_t st);
// matrix-core path for 5+ rows (mfma_gemv.hip); launch_linear / launch_swiglu route to it when cfg == 0
bool mfma_linear_applies(const LinearArgs& a);
int launch_linear_mfma(const LinearArgs& a, hipStream_t st);
bool mfma_swiglu_applies(const SwigluArgs& a);
int launch_swiglu_mfma(const SwigluArgs& a, hipStream_t st);
int launch_swiglu(const SwigluArgs& a, int cfg, hipStream_t st);

// group-wise int4 weights (q4_gemv.hip): one matrix (linear) or the gate/up pair of the SwiGLU
struct Q4Args {
  const uint16_t* x; int64_t ldx; int64_t up_off;   // [B, >= K] bf16; the second matrix reads x + up_off
  const uint8_t* qw[2]; int64_t ldq;                // [N, ldq] bytes, two columns per byte (even column low nibble)
  const uint16_t* sc[2]; const int16_t* zr[2]; int64_t ldg;   // fp16 scales / int16 zero points [N, ldg]
  int group;                                        // columns per group (power of two >= 32), <= 0 or >= K: one per row
  const uint16_t* bias; const uint16_t* norm_w; float eps;
  const uint16_t* res; int64_t ldres;
  uint16_t* y; int64_t ldy;
  int B, N, K, nmat, mode;
  int dt = 0;                                       // element type of x, bias, norm_w, res and y
};
int launch_linear_q4(const Q4Args& a, hipStream_t st);
int launch_dequant_q4(const uint8_t* qw, int64_t ldq, const uint16_t* sc, const int16_t* zr, int64_t ldg, int group, uint16_t* w,
                      int64_t ldw, int N, int K, int dt, hipStream_t st);
int launch_qkv(const QkvArgs& a, int cfg, hipStream_t st);
int launch_rmsnorm(const uint16_t* x, int64_t ldx, const uint16_t* w, float eps, uint16_t* y, int64_t ldy, int rows,
                   int K, int dt, hipStream_t st);
int launch_attn_decode(const AttnDecodeArgs& a, hipStream_t st);
int launch_kv_append(const KvAppendArgs& a, hipStream_t st);
size_t attn_decode_ws_floats(int B, int H, int nsplit, int Dh);

}  // namespace fsvd

// persistent decode step (decode_step.hip); the argument structs are part of the public header
struct fsvd_phase;
struct fsvd_step_state;
namespace fsvd {
int decode_step_workgroups();
int prepare_decode_step(fsvd_phase* host_phases, int nph, int nwg);
int validate_decode_step(const fsvd_phase* host_phases, int nph, int nwg);
int decode_step_build(const fsvd_phase* host_phases, int nph);   // 0 bf16, 1 with int4 phases, 2 with the composed form's phases
int launch_decode_step(const fsvd_phase* dev_phases, int nph, fsvd_step_state* state, unsigned long long* trace,
                       int trace_stride, int build, hipStream_t stream);
}  // namespace fsvd

