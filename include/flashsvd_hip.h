/*
 * libflashsvd_hip — C ABI of the MI355X (gfx950) low-rank decode kernels.
 *
 * Conventions
 *   - every pointer is a device pointer unless it says "host";
 *   - tensors are bf16 (uint16 bit patterns) unless a dtype argument says otherwise;
 *   - leading dimensions / strides are in ELEMENTS;
 *   - `stream` is a hipStream_t (NULL = the default stream); launches are asynchronous;
 *   - the return value is 0 on success and a negative FSVD_ERR_* code otherwise, with a
 *     human-readable message available from fsvd_last_error() (thread-local);
 *   - no entry point allocates or frees device memory: scratch is passed in by the caller.
 *
 * Reference paths cited below are relative to the FlashSVD checkout.
 */
#ifndef FLASHSVD_HIP_H_
#define FLASHSVD_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FSVD_OK 0
#define FSVD_ERR_BAD_SHAPE (-1)
#define FSVD_ERR_BAD_ALIGN (-2)
#define FSVD_ERR_BAD_DTYPE (-3)
#define FSVD_ERR_NULL_PTR (-4)
#define FSVD_ERR_LAUNCH (-5)
#define FSVD_ERR_WORKSPACE (-6)

/* dtype codes for the entry points that take one (the reference kernels switch on
 * USE_BF16 / USE_FP32, kernels/attn/decode/densekv_reconstruct_triton.py:427-428) */
#define FSVD_BF16 0
#define FSVD_FP16 1
#define FSVD_FP32 2

int fsvd_version(void);
const char* fsvd_last_error(void);

/* Optional scratch for the projections of 17..127 rows, and of 3..16 rows when the matrix has fewer than 2048 rows
 * (fsvd_linear, fsvd_swiglu_linear): with it they run on 32-row tiles and split K over several workgroups per tile
 * (fp32 partial tiles and arrival counters live in this buffer; the sum is taken in a fixed order, so results do not
 * depend on timing).
 * The library never allocates device memory: the caller owns `ws` (device memory of the current device, 256-byte
 * aligned, `bytes` >= 1 MiB to be of use, 64 MiB covers every shape of a 7B model) and keeps it alive until it
 * registers another buffer or NULL.  The first 64 KiB are cleared here, on `stream`.  One buffer per device; launches
 * that use it must be ordered on one stream (two concurrent projections would share the counters).  Without a
 * registered buffer the same entry points run unsplit.  No counterpart in the reference (torch.matmul picks its own
 * split-K workspace inside hipBLASLt). */
int fsvd_set_workspace(void* ws, size_t bytes, void* stream);

/* The fused product path below (projections, SwiGLU pair, q / k / v of the current token, attention over the dense
 * cache, RMSNorm, head expansion and prompt attention) computes in the 16-bit type its `dtype` argument names,
 * FSVD_BF16 or FSVD_FP16: every tensor of a call is of that type ("bf16" in the formulas stands for it), sums are
 * fp32, roundings are to nearest even at the same points in both.  The reference picks the type from its inputs the
 * same way (kernels/attn/decode/densekv_reconstruct_triton.py:427-428; fp16 is the default of its dense cache,
 * runtime/cache/attn_dense_kv.py:26, and the fallback of scripts/demo_support/api.py:161-165).  So does the rank-space
 * decode attention (fsvd_attn_decode_rankkv; fsvd_rankkv_append copies 16-bit patterns of either type).  The
 * persistent decode step takes its type from its phase list (FSVD_WBITS_FP16, FSVD_WBITS_Q4_FP16); the int4 entries
 * take activations of either type. */

/* y[b,n] = (res[b,n] +) bf16( W[n,:] . norm(x[b,:]) (+ bias[n]) ),  W is an nn.Linear weight [N,K].
 * norm_w != NULL fuses the RMSNorm of x (w * bf16(x * rsqrt(mean(x^2)+eps))) in front.
 * Replaces the factor GEMVs the reference issues through torch: rank projection
 * `hidden @ packed_qkv_rank` (benchmark/attn/decode_compare.py:1538), `o_u_proj(o_v_proj(.))`
 * (utils/model_utils.py:332-341), `up_v_proj/gate_v_proj` (benchmark/mlp/bench_svd_llama_decode_graph.py:133),
 * phase-2 `matmul(S, DownU)` (kernels/mlp/decode/dual_split_triton.py:719-721) and RMSNorm
 * (benchmark/mlp/bench_svd_llama_decode_graph.py:78-83).  cfg = 0 picks the tiling. */
int fsvd_linear(const void* x, int64_t ldx, const void* W, int64_t ldw, const void* bias,
                const void* norm_w, float eps, const void* res, int64_t ldres,
                void* y, int64_t ldy, int B, int N, int K, int cfg, int dtype, void* stream);

/* h[b,n] = silu(gate_u[n,:] . p[b,0:R]) * (up_u[n,:] . p[b,up_off:up_off+R]),  gate_u/up_u [D,R].
 * mode 0 rounds like a chain of bf16 nn.Linear modules, mode 1 like the fused reference kernel
 * (h = bf16(silu(g32)*u32), kernels/mlp/decode/dual_split_triton.py:207). */
int fsvd_swiglu_linear(const void* p, int64_t ldp, int64_t up_off, const void* gate_u, const void* up_u,
                       int64_t ldw, void* h, int64_t ldh, int B, int D, int R, int mode, int cfg, int dtype, void* stream);

/* The same projection on group-wise int4 weights: y[b,n] = (res[b,n] +) round( sum_k norm(x)[b,k] * s[n,g(k)] *
 * (q[n,k] - z[n,g(k)]) (+ bias[n]) ).  qweight [N, ldq] bytes holds two columns per byte (even column in the low
 * nibble), scales fp16 and zeros int16 are [N, ldg] with one entry per group_size columns (a power of two >= 32;
 * <= 0 means one group per row): the buffers of the reference's PackedQuantLinear as they are
 * (src/quant/packed_quant_linear.py:18-26 packing, :126-172 quantisation, :284-299 dequantisation, :301-312 forward).
 * The sum runs on the un-rounded s * (q - z) in fp32, which the reference rounds to the activation type first.
 * K must be a multiple of 256; B rows go in slices of four.  dtype names the type of x, bias, norm_w, res and y. */
int fsvd_linear_q4(const void* x, int64_t ldx, const void* qweight, int64_t ldq, const void* scales, const void* zeros,
                   int64_t ldg, int group_size, const void* bias, const void* norm_w, float eps, const void* res,
                   int64_t ldres, void* y, int64_t ldy, int B, int N, int K, int dtype, void* stream);

/* w[n,k] = round(s[n,g(k)] * (q[n,k] - z[n,g(k)])): PackedQuantLinear.dequantize for 4 bits and a result of type dtype
 * (src/quant/packed_quant_linear.py:284-299); any K and group size. */
int fsvd_dequant_q4(const void* qweight, int64_t ldq, const void* scales, const void* zeros, int64_t ldg, int group_size,
                    void* w, int64_t ldw, int N, int K, int dtype, void* stream);

/* fsvd_swiglu_linear on int4 gate_u / up_u [D, R] (same layout for both; rounding modes as above). */
int fsvd_swiglu_linear_q4(const void* p, int64_t ldp, int64_t up_off, const void* gate_q, const void* gate_scales,
                          const void* gate_zeros, const void* up_q, const void* up_scales, const void* up_zeros, int64_t ldq,
                          int64_t ldg, int group_size, void* h, int64_t ldh, int B, int D, int R, int mode, int dtype, void* stream);

/* Current-token q/k/v from packed rank coefficients p[b] = [Pq|Pk|Pv] and nn.Linear-layout
 * u_proj weights, rotate-half RoPE on q and k at positions[b] (eager bf16 arithmetic), q to
 * q_out [B,H,Dh], k/v appended to the dense caches [B,S,Hk,Dh] at positions[b].
 * Fuses reconstruct_qkv_token_shared* (kernels/attn/decode/densekv_reconstruct_triton.py:464-659)
 * with the rotary + cache write the reference leaves to flash_attn_with_kvcache
 * (runtime/attn/decode_registry.py:177-211) and prepare_fa2_direct_write_step
 * (runtime/cache/attn_dense_kv.py:258-311).  cos/sin [rope_len, Dh/2] may be NULL (no rotation). */
int fsvd_qkv_rope_append(const void* p, int64_t ldp, const void* q_u, int64_t ldq, const void* k_u, int64_t ldk,
                         const void* v_u, int64_t ldv, const void* cos, const void* sin, int rope_len,
                         const int32_t* positions, void* q_out, void* k_cache, void* v_cache,
                         int64_t sc_b, int64_t sc_s, int64_t sc_h,
                         int B, int H, int Hk, int Dh, int Rq, int Rk, int Rv, int S, int cfg, int dtype, void* stream);

/* Bytes of scratch fsvd_attn_decode_densekv needs for nsplit > 1: a 256 KiB block of int32 arrival
 * counters followed by the fp32 partials.  The workspace must be zero-filled before its first use;
 * every call leaves the counters at zero, so it can be reused by later calls of any shape that fits. */
size_t fsvd_attn_decode_workspace_bytes(int B, int H, int Dh, int nsplit);

/* Single-query attention over a dense KV cache; the role of flash-attn's
 * flash_attn_with_kvcache in the reference (runtime/attn/decode_registry.py:177-211,
 * benchmark/attn/decode_compare.py:530-566).  q [B,H,Dh]; caches [B,S,Hk,Dh];
 * if k_new/v_new [B,Hk,Dh] are given they are rotated (cos/sin given) and written at
 * cache_seqlens[b] first, then attention runs over cache_seqlens[b]+1 keys; otherwise over
 * cache_seqlens[b]+seqlen_add keys.  cos/sin != NULL also rotates q at cache_seqlens[b].
 * softmax scale = 1/sqrt(Dh) when scale <= 0.  out [B,H,Dh]. */
int fsvd_attn_decode_densekv(const void* q, int64_t sq_b, int64_t sq_h,
                             void* k_cache, void* v_cache, int64_t sc_b, int64_t sc_s, int64_t sc_h,
                             const void* k_new, int64_t sk_b, int64_t sk_h, const void* v_new, int64_t sv_b, int64_t sv_h,
                             const int32_t* cache_seqlens, int seqlen_add,
                             const void* cos, const void* sin, int rope_len,
                             void* out, int64_t so_b, int64_t so_h,
                             void* workspace, size_t workspace_bytes,
                             int B, int H, int Hk, int Dh, int S, int nsplit, float scale, int dtype, void* stream);

/* fsvd_attn_decode_densekv with the split scratch held by the library itself: no workspace argument and no device
 * allocation anywhere in the call.  No counterpart in the reference; it exists for callers that cannot allocate
 * or size a workspace — code under HIP stream capture, tight serving loops, harnesses that forbid hipMalloc.  The
 * scratch is one fixed array of fsvd_attn_decode_densekv_static_max_bytes() (4 MiB) per GPU, held until the process
 * ends; a call whose fsvd_attn_decode_workspace_bytes(B, H, Dh, nsplit) exceeds it returns FSVD_ERR_WORKSPACE.  Every
 * call on a GPU shares that GPU's array: calls that overlap on one GPU (two streams, two threads) race; calls ordered
 * on one stream are safe, and each call clears the arrival counters it uses before its kernels run.  Results are
 * bit-identical to fsvd_attn_decode_densekv on the same arguments. */
size_t fsvd_attn_decode_densekv_static_max_bytes(void);
int fsvd_attn_decode_densekv_static(const void* q, int64_t sq_b, int64_t sq_h,
                                    void* k_cache, void* v_cache, int64_t sc_b, int64_t sc_s, int64_t sc_h,
                                    const void* k_new, int64_t sk_b, int64_t sk_h, const void* v_new, int64_t sv_b, int64_t sv_h,
                                    const int32_t* cache_seqlens, int seqlen_add,
                                    const void* cos, const void* sin, int rope_len,
                                    void* out, int64_t so_b, int64_t so_h,
                                    int B, int H, int Hk, int Dh, int S, int nsplit, float scale, int dtype, void* stream);

/* y = w * bf16(x * rsqrt(mean(x^2)+eps)) over rows of length K.
 * benchmark/mlp/bench_svd_llama_decode_graph.py:78-83. */
int fsvd_rmsnorm(const void* x, int64_t ldx, const void* w, float eps, void* y, int64_t ldy, int rows, int K, int dtype,
                 void* stream);

/* ---------------------------------------------------------------------------------------------
 * Reference operand layouts ("x @ W", W is [K, N]).  dtype is FSVD_BF16 / FSVD_FP16 / FSVD_FP32;
 * accumulation is fp32 with one rounding at the store.  Workspaces: bytes from the matching
 * *_workspace_bytes call; the first use needs the workspace zero-filled, later calls keep it valid.
 * ------------------------------------------------------------------------------------------- */

/* y[b,:] = x[b,:] @ W (+ bias).  Replaces torch.matmul(hidden, packed_qkv_rank)
 * (benchmark/attn/decode_compare.py:1538), the three matmuls of
 * reconstruct_qkv_token_shared_prepacked (kernels/attn/decode/densekv_reconstruct_triton.py:739-741)
 * and phase 2 of the dual-split MLP, matmul/addmm(S, DownU) (kernels/mlp/decode/dual_split_triton.py:623,721).
 * x_fp32 / out_fp32: activations / result held in fp32 while W is `dtype`.  bias_post != 0 adds the
 * bias after the product has been rounded (`Q = Q + bq`, densekv_reconstruct_triton.py:747-758). */
size_t fsvd_xw_linear_workspace_bytes(int B, int K, int N, int dtype);
int fsvd_xw_linear(const void* x, int64_t sx_b, int64_t sx_k, int x_fp32, const void* W, int64_t sw_k,
                   const void* bias, int bias_post, void* y, int64_t sy_b, int out_fp32,
                   int B, int K, int N, int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* Current-token reconstruction Q[b,h,:] = Pq[b,(h),:] @ Vq[h] (+ bq[h]) and the same for K, V over
 * Hk heads.  One entry point for the three reference kernels: headwise P [B,H,R] (sP*_h = R stride),
 * shared P [B,R] (sP*_h = 0) and hetero ranks (Rq, Rk, Rv differ).
 * kernels/attn/decode/densekv_reconstruct_triton.py:11-357 (kernels), :360-659 (wrappers).
 * Bases V* are [heads, R, Dh] with unit stride along Dh; biases [heads, Dh] or NULL. */
size_t fsvd_reconstruct_qkv_workspace_bytes(int B, int H, int Hk, int Dh, int Rq, int Rk, int Rv, int dtype);
int fsvd_reconstruct_qkv_token(const void* Pq, int64_t sPq_b, int64_t sPq_h, int64_t sPq_r,
                               const void* Pk, int64_t sPk_b, int64_t sPk_h, int64_t sPk_r,
                               const void* Pv, int64_t sPv_b, int64_t sPv_h, int64_t sPv_r,
                               const void* Vq, int64_t sVq_h, int64_t sVq_r,
                               const void* Vk, int64_t sVk_h, int64_t sVk_r,
                               const void* Vv, int64_t sVv_h, int64_t sVv_r,
                               const void* bq, int64_t sbq_h, const void* bk, int64_t sbk_h, const void* bv, int64_t sbv_h,
                               void* Q, int64_t sQ_b, int64_t sQ_h, void* K, int64_t sK_b, int64_t sK_h,
                               void* V, int64_t sV_b, int64_t sV_h,
                               int B, int H, int Hk, int Dh, int Rq, int Rk, int Rv, int dtype,
                               void* workspace, size_t workspace_bytes, void* stream);

/* Dual-split low-rank SwiGLU MLP on the reference operands: PUp, PGate [T,R] (row strides given),
 * GateU, UpU [R,D], DownV [D,R], DownU [R,Hd], optional b2 [Hd]; Y [T,Hd].
 *   h = dtype(silu(PGate@GateU) * (PUp@UpU));  S = sum over D tiles of bd rows of h[:,tile] @ DownV[tile,:];
 *   Y = dtype(S) @ DownU (+ b2).
 * variant 1: tile partials pass through a workspace of `dtype` (or fp32 when partials_fp32 != 0) before
 *            the sum (flashsvd_mlp_dual_split_triton_v1, kernels/mlp/decode/dual_split_triton.py:535-624);
 * variant 2: fp32 partials summed into S, which is then rounded (v2 / v2_sm80 / pcat_s, :627-855 and
 *            dual_split_triton_pcat_s.py:123-218); S_out, if given, receives the fp32 S [T,R];
 * variant 3: tile partials rounded to dtype, Y accumulated in fp32 from them and rounded once, b2 added
 *            afterwards in dtype (v3, dual_split_triton.py:427-532,858-966).
 * The summation over D tiles is in tile order (deterministic), unlike the reference's atomics. */
size_t fsvd_mlp_dual_split_workspace_bytes(int T, int R, int D, int Hd, int dtype, int bd);
int fsvd_mlp_dual_split(const void* PUp, int64_t sPUp_t, const void* PGate, int64_t sPGate_t,
                        const void* GateU, int64_t ldGateU, const void* UpU, int64_t ldUpU,
                        const void* DownV, int64_t ldDownV, const void* DownU, int64_t ldDownU, const void* b2,
                        void* Y, int64_t ldY, float* S_out, int T, int R, int D, int Hd, int dtype,
                        int variant, int bd, int partials_fp32, void* workspace, size_t workspace_bytes, void* stream);

/* Single-query attention over a rank-space KV cache (pre-RoPE coefficients Pk, Pv [B,S,R] shared
 * by all heads; runtime/cache/attn_legacy_sparse_kv.py:22-35).  K tiles are rebuilt in-kernel as
 * Pk @ k_u[h]^T on the matrix cores and rotated at absolute key positions, the softmax weights are
 * applied to Pv in rank space and one product with v_u[h] finishes each head.  Semantics of the
 * reference's streaming decode, benchmark/attn/decode_compare.py:675-750, and of the (absent) fused
 * kernels behind flashsvd_attn_decode_packed (:823-948): q [B,H,Dh] is the current token's query
 * (rotate_q != 0 rotates it at position n_keys-1), k_u / v_u are nn.Linear-layout u_proj weights
 * [Hk*Dh, R] (= per-head bases V[h][r][d] = u[h*Dh+d][r]), workspaces are the reference's split-K
 * buffers M, L [B,H,nsplit] and Acc [B,H,nsplit,Rv] (fp32), n_keys = cache_seqlens[b] + seqlen_add.
 * spk_h / spv_h are the kv-head strides of head-wise coefficient caches [B,S,Hk,R] (0 when shared).
 * bf16 only; head_dim 128; ranks multiples of 8, Rv <= 2048.
 * Long caches shared by the heads (spv_h == 0, S >= 256, B*H*ceil64(S) >= 2^17) can run as score, softmax and
 * accumulation launches (same results up to the order of fp32 sums) when the caller passes `scores`, a buffer of
 * fsvd_attn_decode_rankkv_scores_bytes(B, H, S, 1) bytes that holds the scores of the call; with scores == NULL, or for a
 * shape for which that size is 0, the call is one kernel + merge.  Which form runs therefore depends on the arguments
 * alone; the buffer belongs to the call, so calls on different streams need different buffers. */
size_t fsvd_attn_decode_rankkv_scores_bytes(int B, int H, int S, int shared_by_heads);
int fsvd_attn_decode_rankkv(const void* q, int64_t sq_b, int64_t sq_h,
                            const void* pk_cache, int64_t spk_b, int64_t spk_s, int64_t spk_h,
                            const void* pv_cache, int64_t spv_b, int64_t spv_s, int64_t spv_h,
                            const void* k_u, int64_t ldku, const void* v_u, int64_t ldvu, const void* bv,
                            const void* cos, const void* sin, int rope_len, int rotate_q,
                            const int32_t* cache_seqlens, int seqlen_add,
                            float* ws_m, float* ws_l, float* ws_acc,
                            void* out, int64_t so_b, int64_t so_h,
                            int B, int H, int Hk, int Dh, int S, int Rk, int Rv, int nsplit, float scale,
                            float* scores, size_t scores_bytes, int dtype, void* stream);

/* The packed rank projection of a decoded token with the cache append in its epilogue, for one or two rows:
 * y[b, :] = bf16( W . norm(x[b, :]) ) with W = [q_v; k_v; v_v] ([Rq + Rk + Rv, K], nn.Linear layout), and the Pk | Pv parts
 * of y also stored at pk_cache[b, positions[b], :] / pv_cache[b, positions[b], :] (caches [B,S,R] with strides (sp*_b,
 * sp*_s, 1); a row whose position is outside [0, S) is not appended).  One launch for `hidden @ packed_qkv_rank`
 * (benchmark/attn/decode_compare.py:1538) plus FlashSVDLegacySparseKVCache.update
 * (runtime/cache/attn_legacy_sparse_kv.py:113-169); the same bits as fsvd_linear followed by fsvd_rankkv_append. */
int fsvd_linear_rankkv_append(const void* x, int64_t ldx, const void* W, int64_t ldw, const void* norm_w, float eps, void* y,
                              int64_t ldy, int B, int Rq, int Rk, int Rv, int K, void* pk_cache, int64_t spk_b, int64_t spk_s,
                              void* pv_cache, int64_t spv_b, int64_t spv_s, const int32_t* positions, int S, int dtype,
                              void* stream);

/* One decoded token per batch row into a rank-space cache: pk_cache[b, positions[b], :] = pk[b, :] and the same for pv
 * (FlashSVDLegacySparseKVCache.update with one position per row, runtime/cache/attn_legacy_sparse_kv.py:113-169: two
 * index_copy_ calls there; one launch here).  Caches are [B,S,R] with strides (sp*_b, sp*_s, 1); a row whose position is
 * outside [0, S) is dropped.  bf16; ranks multiples of 8; pointers and strides 16-byte aligned. */
int fsvd_rankkv_append(const void* pk, int64_t ldpk, const void* pv, int64_t ldpv,
                       void* pk_cache, int64_t spk_b, int64_t spk_s, void* pv_cache, int64_t spv_b, int64_t spv_s,
                       const int32_t* positions, int B, int S, int Rk, int Rv, void* stream);

/* Full-sequence low-rank RoPE attention = the role of the fused Triton kernel flashsvd_rope_sdpa
 * (kernels/attn/prefill/rope_sdpa.py:67-248, wrapper FlashSVDRoPEAttention :254-427), as two launches:
 *
 * fsvd_lowrank_expand_heads: y[b, row, head, :] = P[b,m,(head),:] @ u[head*Dh:(head+1)*Dh, :]^T
 *   (+ bias), rounded to bf16, then rotate-half RoPE at position positions[b]+m when cos/sin are given,
 *   stored at row = m (dst_by_position = 0: a query buffer [B,M,H,Dh]) or row = positions[b]+m
 *   (dst_by_position = 1: the dense KV cache [B,S,Hk,Dh]; rows outside [0,dst_rows) are dropped).
 *   P is [B,M,heads,R] with sp_h = 0 for coefficients shared by all heads; u is the nn.Linear-layout
 *   u_proj weight [heads*Dh, R] (per-head basis V[h][r][d] = u[h*Dh+d][r]).  bf16, Dh = 128, R % 8 == 0.
 *
 * fsvd_attn_prefill: out[b,m,h,:] = softmax_n(q[b,m,h,:] . k[b,n,hk,:] * scale + masks) v[b,n,hk,:]
 *   over keys n < q_pos0[b] + M, causal (n <= q_pos0[b] + m) when causal != 0; pad_mask [B,keys] (0 =
 *   masked key), add_mask [B,M,keys] fp32 added to the scaled scores; rows with no visible key give 0
 *   (rope_sdpa.py:195-209,244-246).  q is already rotated; k is the post-RoPE cache. */
int fsvd_lowrank_expand_heads(const void* p, int64_t sp_b, int64_t sp_m, int64_t sp_h, const void* u, int64_t ldu,
                              const void* bias, const void* cos, const void* sin, int rope_len, const int32_t* positions,
                              void* y, int64_t sy_b, int64_t sy_m, int64_t sy_h, int dst_by_position, int dst_rows,
                              int B, int M, int heads, int Dh, int R, int dtype, void* stream);
/* The q, k and v expansions of one prompt pass in one call: the same results as `n` calls of
 * fsvd_lowrank_expand_heads on the same token rows (one per descriptor; `rotate` selects whether that one gets the
 * rotation), and a single launch when every one of them takes the tiled kernel (128 token rows and more, rank a
 * multiple of 64, coefficients shared by the heads).  The reference computes all three inside one kernel as well
 * (rope_sdpa.py:67-248 takes Pq/Vq, Pk/Vk, Pv/Vv together).  n = 1..3. */
typedef struct fsvd_expand_desc {
  const void* p; int64_t sp_b, sp_m, sp_h;   /* rank coefficients [B,M,(heads),R] */
  const void* u; int64_t ldu;                /* [heads*Dh, R] */
  const void* bias;                          /* [heads*Dh] or NULL */
  void* y; int64_t sy_b, sy_m, sy_h;         /* destination [B, rows, heads, Dh] */
  int32_t heads, R;
  int32_t rotate;                            /* 1: rotate-half RoPE with the call's cos / sin */
  int32_t dst_by_position, dst_rows, rsv0;
} fsvd_expand_desc;
int fsvd_lowrank_expand_heads_multi(const fsvd_expand_desc* desc, int n, const void* cos, const void* sin, int rope_len,
                                    const int32_t* positions, int B, int M, int Dh, int dtype, void* stream);
int fsvd_attn_prefill(const void* q, int64_t sq_b, int64_t sq_m, int64_t sq_h,
                      const void* k, const void* v, int64_t sk_b, int64_t sk_s, int64_t sk_h,
                      const int32_t* q_pos0, const uint8_t* pad_mask, int64_t spm_b,
                      const float* add_mask, int64_t sam_b, int64_t sam_q,
                      void* out, int64_t so_b, int64_t so_m, int64_t so_h,
                      int B, int M, int H, int Hk, int Dh, int S, int causal, float scale, int dtype, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Persistent decode step (batch 1): ONE launch walks a caller-built list of phases — embedding row,
 * low-rank projections with fused RMSNorm / residual / SwiGLU, q/k/v head expansion with RoPE and
 * cache append, split-KV attention and its merge, lm_head and greedy argmax — on one workgroup per
 * compute unit.  Workgroups hand activations to each other through "tagged" vectors: every 32-bit
 * word carries a bf16 value and a 16-bit tag (fp32 partials: 64-bit words with a 32-bit tag) that
 * changes with every use of the buffer, so a consumer polls the data itself and no grid barrier, L2
 * write-back or counter is needed; while a workgroup waits, the first weights of its next phase are
 * already in flight.  It replaces, for greedy batch-1 decoding, the per-token module walk of
 * utils/evaluator.py:39-82 (_manual_llama_decode_step) and scripts/demo_support/api.py:238-322 together
 * with the per-layer operators listed above; arithmetic and rounding points are those of the
 * stand-alone entry points (fsvd_linear, fsvd_swiglu_linear mode 0/1, fsvd_qkv_rope_append,
 * fsvd_attn_decode_densekv).
 *
 * Rules for the phase list (checked by fsvd_decode_step): every matrix has K % 128 == 0 and at least
 * one row per workgroup; a tagged buffer is written by one phase per step position and must not be
 * written again until a later GEMV phase has consumed a vector that every workgroup helped to write
 * (use separate buffers per role and two alternating hidden-state buffers).  All tagged buffers and
 * the state block start zero-filled.  Polls are bounded: on a time-out the step sets state->err and
 * every workgroup leaves; later launches return immediately until the caller clears err.
 * ------------------------------------------------------------------------------------------- */
#define FSVD_PH_EMBED 0   /* out0[n] = W[0][token, n]                                   (N = hidden)        */
#define FSVD_PH_GEMV 1    /* out0 = epilogue(W[m] . norm(in)), m < nmat; bf16 weights, or int4 when wbits == 4  */
#define FSVD_PH_ATTN 3    /* in = un-rotated [q | k | v] of the current token ((H + 2*Hk) * Dh values, the   */
                          /* output of a GEMV over the row-packed [q_u; k_u; v_u], or of a plain GEMV of that   */
                          /* many rows): rotate-half RoPE on q, k                                            */
                          /* at state->pos, append k, v to the cache, split-KV attention; out0 = partials    */
#define FSVD_PH_MERGE 4   /* out0 = merged attention output from in = partials                               */
#define FSVD_PH_ARGMAX 5  /* token = argmax of the per-workgroup candidates in `in`; advances the state      */

#define FSVD_WBITS_FP16 (-16) /* fsvd_phase.wbits of a GEMV phase whose weights are float16 (see there)                */
#define FSVD_WBITS_Q4_FP16 (-4) /* ... whose weights are int4 and whose activations are float16                         */

#define FSVD_EP_STORE 0   /* out0[n] = bf16(dot)                                                              */
#define FSVD_EP_RESID 1   /* out0[n] = bf16(aux0[n] + bf16(dot))                                              */
#define FSVD_EP_SWIGLU 2  /* nmat = 2: out0[n] = silu(W[0][n].in[0:K]) * (W[1][n].in[K:2K]), rounding `mode`  */
                          /* (shared_in: both over in[0:K])                                                   */
#define FSVD_EP_LOGITS 3  /* plain_out[n] = bf16(dot) and out0[wg] = (best value, best index) of the workgroup */
#define FSVD_EP_F32 4     /* out1[n - rows0] = dot (+ aux2[n - rows0]) as fp32 in a 64-bit tagged word: a sum that a  */
                          /* later phase completes or scales before it is rounded                                */

/* GEMV phase flags.  They exist for the composed form of a low-rank layer, in which RMSNorm is applied as a scalar
 * after the product (norm weights folded into the matrix): W.(x + U.t) = W.x + (W.U).t, so the product with the hidden
 * state x can be taken in an earlier phase that has x staged anyway (as an FSVD_PF_NOWAIT phase behind the publication
 * of that phase's own outputs, where its weight stream hides the hand-off), and the phase that applies U also applies
 * the pre-multiplied W.U and emits the finished sum unrounded (FSVD_PF_SPLIT).  No counterpart in the reference, whose
 * walk (utils/evaluator.py:39-82) launches one operator per projection. */
#define FSVD_PF_NOWAIT 1  /* the input was staged by the previous phase of this workgroup (at in_off): no polling   */
#define FSVD_PF_STAGE2 2  /* `in` holds fp32 sums (64-bit tagged words, nmat * K or 3 * K of them) and in2 the raw   */
                          /* bf16 hidden state they were taken from: staged input = bf16(in * rsqrt(mean(in2^2) +  */
                          /* fparam)) at 0, and in2 itself, unscaled, at in2_off for a following NOWAIT phase     */
#define FSVD_PF_SPLIT 4   /* two row groups with their own epilogues and outputs, see rows0                       */
#define FSVD_PF_LEAD 8    /* with FSVD_PF_NOWAIT, on a single-matrix FSVD_EP_F32 phase: the phase only streams (its   */
                          /* input is a vector that an earlier FSVD_PF_STAGE2 staging left at in_off and nothing has  */
                          /* overwritten since); it neither polls nor publishes, its sums wait in the workgroup's     */
                          /* partial buffer, and the NEXT phase - a plain single-matrix bf16 GEMV, which polls for    */
                          /* its own input only behind that stream - publishes them with its own.  The slab must     */
                          /* fill whole windows of loads.                                                            */

typedef struct fsvd_tagbuf {
  void* ptr;              /* uint32 [len] (bf16 payload) or uint64 [len] (fp32 / candidate payload)           */
  int32_t uses_per_step;  /* how many phases of one step write this buffer                                    */
  int32_t use;            /* which of those uses this phase writes (out*) or reads (in, aux*)                 */
} fsvd_tagbuf;

typedef struct fsvd_phase {
  int32_t type, epilogue;
  int32_t N, K, nmat, mode;     /* rows per matrix, row length, matrices, SwiGLU rounding mode; the staged     */
                                /* input has nmat * K elements.  EMBED: K = rows of the table (0: unchecked);  */
                                /* a token outside [0, K) reads row 0 and sets state->err                      */
  int32_t H, Hk, Dh;            /* on a GEMV, H > 0 marks the q | k | v head expansion: N = (H + 2*Hk) * Dh    */
                                /* rows in three groups that read in[0:K], in[K:2K], in[2K:3K]                 */
  union { int32_t nsplit;       /* ATTN, MERGE: key splits per head                                            */
          int32_t rows0; };     /* GEMV with FSVD_PF_SPLIT: rows [0, rows0) take `epilogue` into out0, rows    */
                                /* [rows0, N) take FSVD_EP_F32 into out1 (+ aux2)                              */
  union { int32_t rope_len;     /* ATTN: rows of cos / sin                                                     */
          int32_t in_off; };    /* GEMV: element offset of this phase's input in the workgroup's staging area  */
  union { int32_t S;            /* ATTN: cache rows                                                            */
          int32_t in2_len; };   /* GEMV with FSVD_PF_STAGE2: elements of in2                                   */
  float fparam;                 /* GEMV with norm_w or FSVD_PF_STAGE2: RMSNorm eps; ATTN: softmax scale        */
  int32_t flags;                /* GEMV: FSVD_PF_* bits                                                        */
  const void* W[3];             /* nn.Linear-layout weights [N, K] (EMBED: table [V, N]); W[2] unused         */
  const void* norm_w;           /* RMSNorm weight over `in` or NULL                                            */
  union {
    struct { const void* cos; const void* sin;     /* ATTN: [rope_len, Dh/2]                                   */
             void* k_cache; void* v_cache; };      /* ATTN: batch row of the dense cache, [S, Hk, Dh], strides sc_s, sc_h */
    struct { fsvd_tagbuf aux2;                     /* GEMV: fp32 addend of the FSVD_EP_F32 rows (ptr NULL: none) */
             fsvd_tagbuf out1; };                  /* GEMV: fp32 output of the FSVD_EP_F32 rows                */
  };
  union { int64_t sc_s;         /* ATTN: cache stride between tokens (elements)                                */
          int32_t in2_off; };   /* GEMV with FSVD_PF_STAGE2: element offset at which in2 is staged             */
  int64_t sc_h;                 /* ATTN: cache stride between heads                                            */
  void* plain_out;              /* EP_LOGITS: bf16 logits [N]; ARGMAX: int64 token log indexed by state->step */
  fsvd_tagbuf in, aux0;         /* aux0: residual of EP_RESID                                                  */
  fsvd_tagbuf in2;              /* GEMV with FSVD_PF_STAGE2: the raw hidden state behind `in` (see the flag)   */
  fsvd_tagbuf out0;
  /* GEMV over group-wise int4 weights (wbits == 4, or FSVD_WBITS_Q4_FP16 in a float16 step; 0 or 16 = bf16): W[m] is
   * the packed matrix [N, K/2] bytes (two columns per byte, even column in the low nibble, as
   * PackedQuantLinear.qweight); qsz[m] is uint32 [N, ldg] with the fp16 scale bits of a group in the low half and
   * (zero point + 128) in the high half ((zero point + 16) in a float16 step); a group is 32 << gshift columns.  K % 256 == 0.  Arithmetic as fsvd_linear_q4: y = sum_g s_g * sum_k x_k (q_k - z_g), fp32. */
  const void* qsz[2];
  int32_t ldg, gshift, wbits;   /* wbits also names the element type of a step: FSVD_WBITS_FP16 (FSVD_WBITS_Q4_FP16 for an   */
                                /* int4 phase) in EVERY GEMV phase of a list makes it a float16 step (vectors, tables,       */
                                /* caches and 16-bit weights float16)                                                        */
  int32_t shared_in;            /* nmat == 2: both matrices read the same K-long input (a dense gate / up pair) instead   */
                                /* of in[0:K] and in[K:2K]                                                                 */
  /* derived by fsvd_decode_step_prepare (do not fill by hand): work items (rows, merge outputs) are
   * dealt as share_q per workgroup plus one more for the first share_r workgroups; m_kp is the 32-bit
   * reciprocal of K/8 and dk = (threads per workgroup) mod (K/8) */
  int32_t share_q, share_r;
  uint32_t m_kp;
  int32_t dk;
} fsvd_phase;

typedef struct fsvd_step_state {
  int32_t epoch;      /* advanced by every completed step; seeds the tags                                     */
  int32_t err;        /* 0 ok; else 1 + index of the phase whose input never arrived, of the EMBED phase that */
                      /* met a token outside its table, or of the ARGMAX phase that found no comparable logit */
  int32_t pos;        /* position of the token being decoded = number of keys already in the cache            */
  int32_t step;       /* tokens generated so far (index into the token log)                                   */
  int64_t token;      /* input token of the next step (written by ARGMAX)                                     */
  int32_t err_wg;     /* workgroup that raised err                                                            */
  int32_t spin_limit; /* polls before a workgroup gives up; 0 = default (about a second)                       */
} fsvd_step_state;

/* Workgroups the step kernel runs with on the current device (one per compute unit), or 0 with fsvd_last_error() when
 * the device cannot hold one workgroup of the kernel per compute unit (the grid must be co-resident: workgroups wait
 * for each other's results).  While a step runs nothing else may execute on the device; a step that is starved of
 * compute units ends by its spin limit with state->err set. */
int fsvd_decode_step_workgroups(void);
/* Fill the derived fields of a host-side phase list for `workgroups` workgroups (call before uploading it). */
int fsvd_decode_step_prepare(fsvd_phase* phases_host, int nphase, int workgroups);
/* The host-side check of fsvd_decode_step alone (no launch): 0, or a negative status with fsvd_last_error(). */
int fsvd_decode_step_validate(const fsvd_phase* phases_host, int nphase, int workgroups);
/* phases_dev: the list in device memory; phases_host: the same list in host memory (validated on every
 * call unless validate == 0; it also tells the launcher which build of the kernel the list needs — plain bf16, with
 * the int4 code, or with the code of the composed form — so it may be NULL only for plain bf16 lists: a build that
 * meets a phase it was not compiled for raises state->err);
 * state: device.  Launch is asynchronous on `stream`. */
int fsvd_decode_step(const fsvd_phase* phases_dev, const fsvd_phase* phases_host, int nphase,
                     fsvd_step_state* state, int validate, void* stream);
/* The same step with per-phase time stamps (the hipEvent-per-module decode profiler of the reference,
 * utils/evaluator.py:553-689, cannot see inside one launch): workgroups 0, wg_stride, 2*wg_stride, ...
 * write trace[(wg / wg_stride) * nphase * 4 + phase * 4 + k], k = 0 phase entered, 1 input staged,
 * 2 weights consumed, 3 epilogue done, in ticks of the 100 MHz device wall clock.  The list must have
 * passed fsvd_decode_step's validation before. */
int fsvd_decode_step_trace(const fsvd_phase* phases_dev, const fsvd_phase* phases_host, int nphase, fsvd_step_state* state,
                           uint64_t* trace, size_t trace_words, int wg_stride, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLASHSVD_HIP_H_ */
