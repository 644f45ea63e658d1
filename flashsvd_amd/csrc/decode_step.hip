// Persistent batch-1 decode step: one workgroup per compute unit walks a list of phases.
//
// Hand-off between workgroups is by "tagged" vectors: a producer stores (tag << 16 | bf16) words with
// write-through agent-scope stores, a consumer polls the words it needs with agent-scope loads until
// every tag matches the tag expected for this use of the buffer.  Tags advance with every use, so stale
// contents never match, and there is no barrier object, counter or L2 write-back on the path.  Before a
// workgroup starts polling for the input of a phase it has already requested the first kU 16-byte
// pieces per lane of that phase's weights, so the HBM stream keeps running while the activations travel.
//
// Weight walk: a workgroup owns a slab of whole rows (the same rows of one or two matrices); the slab is
// cut into 16-byte pieces dealt to the lanes in address order (fully coalesced); 16 consecutive lanes
// form a chunk (128 elements of one row, K % 128 == 0) whose partial dot product is folded with DPP and
// parked in LDS; row sums add the chunks in a fixed order, so results do not depend on timing.
//
// At this scale (a phase lasts 3-10 us) instruction issue is a first-order cost: a wave retires one
// vector instruction per ~4 cycles, so every hundred instructions on the critical path of a phase is
// ~0.2 us.  Hence: descriptors travel in a VGPR and are read with readlane where needed, work splits and
// reciprocals are precomputed on the host, per-piece address arithmetic is incremental, and waves that
// own no output rows skip the epilogue.
#include <algorithm>
#include <cstddef>
#include <type_traits>
#include <vector>

#include "../../include/flashsvd_hip.h"
#include "common.hpp"
#include "kernels.hpp"

namespace fsvd {

constexpr int kT = 512;                 // threads per workgroup
constexpr int kU = 4;                   // 16-byte weight pieces in flight per lane (rolling register window).  Measured 2 / 4 / 6 / 8 /
                                        // 10 / 12: 451 / 489 / 478 / 471 / 469 / 452 tok/s on the 7B shape: the polls for a phase's
                                        // input queue behind the window requested just before them, so a deep window delays them
constexpr int kUA = kU / 2;             // attention: keys (and values) in flight per 16-lane slot
constexpr int kMaxIn = 16384;           // staged input elements (bf16) per phase
constexpr int kMaxChunks = 8192;        // chunk partials per workgroup per phase
constexpr int kSpinLimit = 1 << 20;     // polls before a workgroup gives up
constexpr int kSlots = kT / 16;         // 16-lane groups = keys in flight per load in the attention phase
constexpr int kMaxPieces = kMaxIn / 32;    // 32-column pieces of a staged input (int4 phases keep their sums)
constexpr int kSzLoads = 3;                // 4-byte loads per lane that bring a slab's scale | zero table (int4 phases)
constexpr int kMaxSz = kSzLoads * kT;      // words of that table: rows x groups x matrices of a workgroup's slab
constexpr size_t kSmemBytes = (size_t)kMaxIn * 2 + (size_t)kMaxChunks * 4 + 256 + (size_t)kMaxPieces * 4 + (size_t)kMaxSz * 4;

// ---------------------------------------------------------------------------------------------
// tagged words
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t tag16_of(int epoch, int ups, int use) {
  return ((uint32_t)epoch * (uint32_t)ups + (uint32_t)use + 1u) & 0xffffu;
}
__device__ __forceinline__ uint32_t tag32_of(int epoch, int ups, int use) {
  return (uint32_t)epoch * (uint32_t)ups + (uint32_t)use + 1u;
}
__device__ __forceinline__ void st_tag16(void* buf, int idx, uint32_t tag, uint32_t bits) {
  __hip_atomic_store(static_cast<uint32_t*>(buf) + idx, (tag << 16) | (bits & 0xffffu), __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_tag64(void* buf, int idx, uint32_t tag, uint32_t payload) {
  __hip_atomic_store(static_cast<uint64_t*>(buf) + idx, ((uint64_t)tag << 32) | payload, __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t ld_coh64(const void* buf, int idx) {
  return __hip_atomic_load(static_cast<const uint64_t*>(buf) + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t ld_coh32(const void* buf, int idx) {
  return __hip_atomic_load(static_cast<const uint32_t*>(buf) + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ int ld_err(const fsvd_step_state* st) {
  return __hip_atomic_load(&st->err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// 16-byte loads through the global (not flat) path: the pointers come out of a descriptor in memory,
// so the compiler cannot tell the address space by itself
typedef const __attribute__((address_space(1))) u32x4_t* gptr16_t;
__device__ __forceinline__ u32x4_t ld_stream(uint64_t base, uint32_t byte_off) {
  return __builtin_nontemporal_load((gptr16_t)(base + byte_off));
}
__device__ __forceinline__ u32x4_t ld_global16(const uint16_t* p) { return *(gptr16_t)(uintptr_t)p; }

// poll one 64-bit word with a 32-bit tag in the high half
__device__ __forceinline__ bool poll_w64(const void* buf, int idx64, uint32_t tag, const fsvd_step_state* st, int limit,
                                         uint32_t& payload) {
  int spins = 0;
  for (;;) {
    const uint64_t v = ld_coh64(buf, idx64);
    payload = (uint32_t)v;
    if ((uint32_t)(v >> 32) == tag) return true;
    if (++spins > limit) return false;
    if ((spins & 1023) == 0 && ld_err(st) != 0) return false;
  }
}

// ---------------------------------------------------------------------------------------------
// A phase descriptor travels in one VGPR per lane (lane k holds 32-bit word k), loaded with a single
// coalesced read two phases ahead of its use; fields come out with readlane where they are needed,
// i.e. without a dependent chain of scalar loads on the critical path.
// ---------------------------------------------------------------------------------------------
constexpr int kDescWords = (int)(sizeof(fsvd_phase) / 4);
static_assert(kDescWords <= 64, "descriptor must fit one wave");
__device__ __forceinline__ uint32_t desc_fetch(const fsvd_phase* phases, int q, int nph) {
  const int lane = threadIdx.x & 63;
  q = q < 0 ? 0 : (q < nph ? q : nph - 1);
  const uint32_t* src = reinterpret_cast<const uint32_t*>(phases + q);
  return src[lane < kDescWords ? lane : 0];
}
#define FSVD_DW(field) ((int)(offsetof(fsvd_phase, field) / 4))
__device__ __forceinline__ uint32_t desc_u32(uint32_t dv, int word) { return (uint32_t)__builtin_amdgcn_readlane((int)dv, word); }
__device__ __forceinline__ uint64_t desc_u64(uint32_t dv, int word) {
  return ((uint64_t)desc_u32(dv, word + 1) << 32) | desc_u32(dv, word);
}
#define DF_I(dv, field) ((int)desc_u32(dv, FSVD_DW(field)))
#define DF_F(dv, field) __uint_as_float(desc_u32(dv, FSVD_DW(field)))
#define DF_P(dv, field) reinterpret_cast<void*>(desc_u64(dv, FSVD_DW(field)))
#define DF_TAG16(dv, tb, epoch) tag16_of(epoch, (int)desc_u32(dv, FSVD_DW(tb) + 2), (int)desc_u32(dv, FSVD_DW(tb) + 3))
#define DF_TAG32(dv, tb, epoch) tag32_of(epoch, (int)desc_u32(dv, FSVD_DW(tb) + 2), (int)desc_u32(dv, FSVD_DW(tb) + 3))

// ---------------------------------------------------------------------------------------------
// GEMV phase: wave-uniform description of this workgroup's slab
//   rows are dealt share_q per workgroup plus one more for the first share_r workgroups
// ---------------------------------------------------------------------------------------------
struct GemvCtx {
  int K, kp, nmat, r0, srows, pps, nsteps, dk;
  int xk;                    // staged elements between the inputs of matrix 0 and matrix 1 (K, or 0 when they share one input)
  int xoff;                  // element offset of the phase's input in the staging area
  uint64_t base0, base1;     // byte addresses of the slab in matrix 0 / 1
  int q4, ldg, gshift;       // int4 weights: a piece is 32 columns; scale | zero words [N, ldg], group = 32 << gshift columns
  uint64_t sz0, sz1;         // byte addresses of the slab's scale | zero rows
};
// wbits of an int4 phase: 4 with bf16 activations, FSVD_WBITS_Q4_FP16 with float16 ones
__host__ __device__ __forceinline__ bool is_q4_bits(int wbits) { return wbits == 4 || wbits == FSVD_WBITS_Q4_FP16; }
// QB: the wbits value of an int4 phase in this build of the kernel (one compare on the walk)
template <bool Q4, int QB>
__device__ __forceinline__ void gemv_ctx(uint32_t dv, int w, GemvCtx& c) {
  c.K = DF_I(dv, K);
  c.q4 = Q4 && DF_I(dv, wbits) == QB;
  c.kp = c.q4 ? c.K >> 5 : c.K >> 3;
  c.nmat = DF_I(dv, nmat);
  c.xk = DF_I(dv, shared_in) ? 0 : c.K;
  c.xoff = DF_I(dv, in_off);
  const int q = DF_I(dv, share_q), r = DF_I(dv, share_r);
  c.r0 = w * q + min(w, r);
  c.srows = q + (w < r ? 1 : 0);
  c.pps = c.srows * c.kp;                       // 16-byte pieces per matrix
  c.nsteps = (c.pps + kT - 1) / kT;             // lane steps per matrix
  c.dk = DF_I(dv, dk);                          // kT % kp
  const uint64_t off = c.q4 ? (uint64_t)(uint32_t)c.r0 * (uint32_t)(c.K >> 1) : (uint64_t)(uint32_t)c.r0 * (uint32_t)c.K * 2u;
  c.base0 = desc_u64(dv, FSVD_DW(W)) + off;
  c.base1 = c.nmat > 1 ? desc_u64(dv, FSVD_DW(W) + 2) + off : c.base0;
  c.ldg = c.gshift = 0;
  c.sz0 = c.sz1 = 0;
  if (c.q4) {
    c.ldg = DF_I(dv, ldg);
    c.gshift = DF_I(dv, gshift);
    const uint64_t so = (uint64_t)(uint32_t)c.r0 * (uint32_t)c.ldg * 4u;
    c.sz0 = desc_u64(dv, FSVD_DW(qsz)) + so;
    c.sz1 = c.nmat > 1 ? desc_u64(dv, FSVD_DW(qsz) + 2) + so : c.sz0;
  }
}
typedef const __attribute__((address_space(1))) uint32_t* gptr32_t;
// plain (cacheable) loads: the scale / zero words are a sixteenth of the weight bytes and are read again every token
__device__ __forceinline__ uint32_t ld_stream32(uint64_t addr) { return *(gptr32_t)addr; }
// first window: slot u holds the piece of step u / NMAT in matrix u % NMAT
template <int NMAT>
__device__ __forceinline__ void gemv_window_addr(const GemvCtx& c, uint64_t (&addr)[kU]) {
  const uint32_t last = (uint32_t)(c.pps - 1);
#pragma unroll
  for (int u = 0; u < kU; ++u) {
    const uint32_t i = min((uint32_t)((u / NMAT) * kT) + threadIdx.x, last);
    addr[u] = ((u % NMAT) ? c.base1 : c.base0) + (i << 4);
  }
}
// the scale | zero words of a slab are contiguous in memory (rows of ldg words, ldg = groups per row): word i of the
// table [matrix][row][group] for lane tid is i = j * kT + tid, j < kSzLoads
__device__ __forceinline__ void gemv_sz_table_addr(const GemvCtx& c, uint64_t (&addr)[kSzLoads]) {
  const uint32_t per = (uint32_t)(c.srows * c.ldg), total = per * (uint32_t)c.nmat;
#pragma unroll
  for (int j = 0; j < kSzLoads; ++j) {
    const uint32_t i = min((uint32_t)(j * kT) + threadIdx.x, total - 1);
    addr[j] = (i >= per ? c.sz1 + ((uint64_t)(i - per) << 2) : c.sz0 + ((uint64_t)i << 2));
  }
}
// consume the window batch by batch; every consumed slot is refilled at once with the piece kU / NMAT
// steps ahead (clamped to the last piece past the end, whose product is dropped).
// GROUPED: the rows form three groups with their own inputs (q, k, v head expansion from [Pq | Pk | Pv]):
// a row at or past g1 / g2 reads the second / third K-long part of the staged vector.
template <class E, int NMAT, bool GROUPED>
__device__ __forceinline__ void gemv_stream(const GemvCtx& c, uint32_t m_kp, int g1, int g2, u32x4_t (&R)[kU], const uint16_t* xs,
                                            float* cp) {
  constexpr int SPB = kU / NMAT;                // steps per batch
  const uint32_t tid = threadIdx.x;
  const uint32_t last = (uint32_t)(c.pps - 1);
  int row = (int)__umulhi(tid, m_kp);           // tid / kp
  int kofs = (int)tid - row * c.kp;             // tid % kp: position of this lane's piece in its row
  row += c.r0;
  const int dq = (int)__umulhi((uint32_t)kT, m_kp);   // rows a lane advances per step (plus the carry of kofs)
  const int cps = c.pps >> 4;                   // chunks per matrix
  const bool lead = (tid & 15) == 0;
  // one batch of the window: products, DPP folds and (REFILL) the loads of the next batch.  The last batch is a copy
  // of the loop body without refills: loads past the slab would sit in the memory pipeline in front of the stores
  // that publish this phase's outputs
  auto batch = [&](int s0, auto refill) {
    constexpr bool REFILL = decltype(refill)::value;
    float d[kU];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      if (s0 + u / NMAT >= c.nsteps) break;     // the rest of the window lies past the slab (uniform)
      const int mat = u % NMAT;
      int xo = mat * c.xk + kofs * 8;
      if (GROUPED) xo += ((row >= g1 ? 1 : 0) + (row >= g2 ? 1 : 0)) * c.K;
      const u32x4_t xv = *reinterpret_cast<const u32x4_t*>(xs + xo);
      d[u] = E::dot8(R[u], xv, 0.f);
      if (REFILL) {
        const uint32_t in = min((uint32_t)((s0 + u / NMAT + SPB) * kT) + tid, last);
        R[u] = ld_stream(mat ? c.base1 : c.base0, in << 4);
      }
      d[u] = row16_sum(d[u]);
      if (mat == NMAT - 1) {
        kofs += c.dk;
        const bool carry = kofs >= c.kp;
        kofs = carry ? kofs - c.kp : kofs;
        if (GROUPED) row += dq + (carry ? 1 : 0);
      }
    }
    if (lead) {
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        if (s0 + u / NMAT >= c.nsteps) break;
        const int i = (s0 + u / NMAT) * kT + (int)tid;
        if (i < c.pps) cp[(u % NMAT) * cps + (i >> 4)] = d[u];
      }
    }
  };
  int s0 = 0;
  for (; s0 + SPB < c.nsteps; s0 += SPB) batch(s0, std::true_type{});
  if (s0 < c.nsteps) batch(s0, std::false_type{});
}
// A leading phase (FSVD_PF_LEAD): a slab whose input this workgroup staged long ago (it sits at an offset of the staging
// area that nothing has overwritten since) is streamed in an iteration of its own that neither polls nor publishes: the
// sums stay in the partial buffer, the window request at the end of the iteration fetches the first pieces of the phase
// behind it, and that phase - which polls for its input only now, when the producers have long published - puts its own
// partial sums behind these and publishes both.  Every step is full and the steps are a multiple of kU (host-checked).
template <class E>
__device__ __forceinline__ void lead_stream(const GemvCtx& a, uint32_t m_kp, u32x4_t (&R)[kU], const uint16_t* xs, float* cp) {
  const uint32_t tid = threadIdx.x;
  const int nA = a.nsteps;
  const int row = (int)__umulhi(tid, m_kp);     // tid / kp
  int kofs = (int)tid - row * a.kp;             // tid % kp
  const bool lead = (tid & 15) == 0;
  // one batch; the last one issues no loads (a copy of the body rather than a condition per load: with a branch in the
  // loop the compiler waits for every load at the top of a batch)
  auto batch = [&](int s0, auto refill) {
    constexpr bool REFILL = decltype(refill)::value;
    float d[kU];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      const u32x4_t xv = *reinterpret_cast<const u32x4_t*>(xs + kofs * 8);
      d[u] = E::dot8(R[u], xv, 0.f);
      if (REFILL) R[u] = ld_stream(a.base0, ((uint32_t)((s0 + u + kU) * kT) + tid) << 4);
      d[u] = row16_sum(d[u]);
      kofs += a.dk;
      kofs = kofs >= a.kp ? kofs - a.kp : kofs;
    }
    if (lead) {
#pragma unroll
      for (int u = 0; u < kU; ++u) cp[((s0 + u) * kT + (int)tid) >> 4] = d[u];
    }
  };
  int s0 = 0;
  for (; s0 + kU < nA; s0 += kU) batch(s0, std::true_type{});
  batch(s0, std::false_type{});
}
// ---------------------------------------------------------------------------------------------
// the same walk over group-wise int4 weights: a 16-byte piece is 32 columns, 8 consecutive lanes form a chunk of
// 256 columns of one row (K % 256 == 0).  No weight becomes a float: OR-ing 0x4300 over a nibble n gives the bf16
// pattern of c + n with c = 128 (float16: 0x4c00 over n << 6, c = 16), the packed dot product multiplies two of them
// with two activations, and with X_p = sum of the piece's activations the piece contributes
// s * (D_p - (z + c) * X_p); the table holds z + c.  The activations sit in LDS in the order the masks
// deliver the nibbles (columns 0,4 | 1,5 | 2,6 | 3,7 of every eight), X_p beside them (stage_store).
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float row8_sum(float v) {
  v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_f32<0x141>(v);  // row_half_mirror
  return v;
}
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
template <class E, int NMAT, bool GROUPED>
__device__ __forceinline__ void gemv_stream_q4(const GemvCtx& c, uint32_t m_kp, int g1, int g2, u32x4_t (&R)[kU], const uint32_t* sztab,
                                               const uint16_t* xs, const float* xsum, float* cp) {
  constexpr int SPB = kU / NMAT;                // steps per batch
  const uint32_t tid = threadIdx.x;
  const uint32_t last = (uint32_t)(c.pps - 1);
  int lrow = (int)__umulhi(tid, m_kp);          // tid / kp: row inside the slab
  int kofs = (int)tid - lrow * c.kp;            // tid % kp: this lane's piece inside its row
  const int dq = (int)__umulhi((uint32_t)kT, m_kp);
  const int cps = c.pps >> 3;                   // chunks per matrix
  const int szper = c.srows * c.ldg;            // table words per matrix
  const bool lead = (tid & 7) == 0;
  auto batch = [&](int s0, auto refill) {
    constexpr bool REFILL = decltype(refill)::value;
    float d[kU];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      if (s0 + u / NMAT >= c.nsteps) break;     // the rest of the window lies past the slab (uniform)
      const int mat = u % NMAT;
      int sel = c.xk ? mat : 0;
      if (GROUPED) sel += (c.r0 + lrow >= g1 ? 1 : 0) + (c.r0 + lrow >= g2 ? 1 : 0);
      const float dp = dot32_q4<E>(R[u], reinterpret_cast<const u32x4_t*>(xs + sel * c.K + kofs * 32));
      const uint32_t sz = sztab[mat * szper + min(lrow, c.srows - 1) * c.ldg + (kofs >> c.gshift)];
      const float sc = (float)__builtin_bit_cast(_Float16, (unsigned short)(sz & 0xffffu));
      const float zz = (float)(int)(sz >> 16);
      d[u] = sc * (dp - zz * xsum[sel * c.kp + kofs]);
      if (REFILL) {
        const uint32_t in = min((uint32_t)((s0 + u / NMAT + SPB) * kT) + tid, last);
        R[u] = ld_stream(mat ? c.base1 : c.base0, in << 4);
      }
      d[u] = row8_sum(d[u]);
      if (mat == NMAT - 1) {
        kofs += c.dk;
        const bool carry = kofs >= c.kp;
        kofs = carry ? kofs - c.kp : kofs;
        lrow += dq + (carry ? 1 : 0);
      }
    }
    if (lead) {
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        if (s0 + u / NMAT >= c.nsteps) break;
        const int i = (s0 + u / NMAT) * kT + (int)tid;
        if (i < c.pps) cp[(u % NMAT) * cps + (i >> 3)] = d[u];
      }
    }
  };
  int s0 = 0;
  for (; s0 + SPB < c.nsteps; s0 += SPB) batch(s0, std::true_type{});
  if (s0 < c.nsteps) batch(s0, std::false_type{});
}
// sum of the chunk partials of one row, computed by an aligned group of 8 lanes (each lane adds every
// eighth chunk, then a three-step DPP butterfly); every lane of the group gets the sum
__device__ __forceinline__ float row_sum8(const float* cp, int row, int cpr) {
  const float* p = cp + row * cpr;
  float t = 0.f;
  for (int c = (int)(threadIdx.x & 7); c < cpr; c += 8) t += p[c];
  t += dpp_f32<0xB1>(t);   // quad_perm [1,0,3,2]
  t += dpp_f32<0x4E>(t);   // quad_perm [2,3,0,1]
  t += dpp_f32<0x141>(t);  // row_half_mirror
  return t;
}

// Staging of the tagged input of a GEMV phase into LDS as packed bf16, RMS-normalised when asked (a normalised input
// fits one round of loads; checked on the host).
// One lane's four consecutive staged values (two packed words, elements 4q .. 4q + 3) into LDS.  For an int4 phase the
// eight values of two neighbouring lanes (columns 0..3 and 4..7 of a group) are stored in the order the nibble masks
// deliver the weights (columns 0,4 | 1,5 | 2,6 | 3,7) and the sum of every 32-column piece (8 lanes) is left in xsum,
// added pairwise: columns, lane pairs, quads, halves.
template <class E>
__device__ __forceinline__ void stage_store_wide(uint16_t* xs, float* xsum, int q, uint32_t w0, uint32_t w1, bool q4) {
  uint2* xs64 = reinterpret_cast<uint2*>(xs);
  if (!q4) { xs64[q] = make_uint2(w0, w1); return; }
  const uint32_t p0 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)w0, 0xB1, 0xF, 0xF, true);   // quad_perm [1,0,3,2]
  const uint32_t p1 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)w1, 0xB1, 0xF, 0xF, true);
  uint2 out;
  if ((threadIdx.x & 1) == 0) {   // columns (0,4), (1,5)
    out.x = (w0 & 0xffffu) | (p0 << 16);
    out.y = (w0 >> 16) | (p0 & 0xffff0000u);
  } else {                        // columns (2,6), (3,7): this lane holds 4..7, its partner 0..3
    out.x = (p1 & 0xffffu) | (w1 << 16);
    out.y = (p1 >> 16) | (w1 & 0xffff0000u);
  }
  xs64[q] = out;                  // q and the lane have the same parity: words 0,1 of the group from the even lane, 2,3 from the odd
  float s = (E::lo(w0) + E::hi(w0)) + (E::lo(w1) + E::hi(w1));
  s += dpp_f32<0xB1>(s);
  s += dpp_f32<0x4E>(s);
  s += dpp_f32<0x141>(s);
  if ((threadIdx.x & 7) == 0) xsum[q >> 3] = s;
}
// The input arrives through 16-byte loads: four tagged values per lane and load.  A workgroup's rate of coherent
// loads is set by their number, not by their bytes (measured on this machine: 44 KB in 1.3 us as 8-byte loads, 0.9 us as
// 16-byte loads, 2.2 us as 4-byte loads, whatever the number of workgroups reading), and every word carries its own tag,
// so a load wider than the atomic unit loses nothing: a word that is torn or stale fails its tag and is polled again.
// The loads are written as instructions: the compiler's forms of a coherent 16-byte load are a volatile access, which
// it follows with a full wait (one round trip per load), or four atomic ones.  All loads of a round AND the wait for
// them are ONE asm statement: the compiler takes an asm statement's outputs as valid the moment it ends, so a load
// left in flight behind its statement may find its destination registers copied, or handed to something else (an
// address), before the data lands.  Outputs are early-clobber: every address is read before the statement ends.
#define FSVD_LDC "global_load_dwordx4 %"
__device__ __forceinline__ void ld_coh128_round(u32x4_t (&v)[2], const uint64_t (&a)[2]) {
  asm volatile(FSVD_LDC "0, %2, off sc0 sc1\n\t" FSVD_LDC "1, %3, off sc0 sc1\n\ts_waitcnt vmcnt(0)"
               : "=&v"(v[0]), "=&v"(v[1])
               : "v"(a[0]), "v"(a[1])
               : "memory");
}
__device__ __forceinline__ void ld_coh128_round(u32x4_t (&v)[5], const uint64_t (&a)[5]) {
  asm volatile(FSVD_LDC "0, %5, off sc0 sc1\n\t" FSVD_LDC "1, %6, off sc0 sc1\n\t" FSVD_LDC "2, %7, off sc0 sc1\n\t"
               FSVD_LDC "3, %8, off sc0 sc1\n\t" FSVD_LDC "4, %9, off sc0 sc1\n\ts_waitcnt vmcnt(0)"
               : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4])
               : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(a[4])
               : "memory");
}
__device__ __forceinline__ void ld_coh128_round(u32x4_t (&v)[8], const uint64_t (&a)[8]) {
  asm volatile(FSVD_LDC "0, %8, off sc0 sc1\n\t" FSVD_LDC "1, %9, off sc0 sc1\n\t" FSVD_LDC "2, %10, off sc0 sc1\n\t"
               FSVD_LDC "3, %11, off sc0 sc1\n\t" FSVD_LDC "4, %12, off sc0 sc1\n\t" FSVD_LDC "5, %13, off sc0 sc1\n\t"
               FSVD_LDC "6, %14, off sc0 sc1\n\t" FSVD_LDC "7, %15, off sc0 sc1\n\ts_waitcnt vmcnt(0)"
               : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7])
               : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(a[4]), "v"(a[5]), "v"(a[6]), "v"(a[7])
               : "memory");
}
#undef FSVD_LDC
template <class E, int NS>
__device__ __forceinline__ bool stage_input_wide(const void* in, int in_len, uint32_t tin, const uint32_t* norm_w, float eps,
                                                 const fsvd_step_state* st, int limit, uint16_t* xs, float* red, bool q4, float* xsum) {
  static_assert(NS == 2 || NS == 8, "ld_coh128_round exists for rounds of 2 and of 8 loads");
  const int tid = threadIdx.x;
  const int nw128 = in_len >> 2;                 // in_len is a multiple of 128
  const bool norm = norm_w != nullptr;
  bool fail = false;
  float ss = 0.f;
  for (int base = 0; base < nw128; base += kT * NS) {
    uint2 nwt[NS];
    if (norm) {   // every slot of the round, index clamped: loads under a condition leave the compiler guarding their registers
#pragma unroll
      for (int j = 0; j < NS; ++j) nwt[j] = reinterpret_cast<const uint2*>(norm_w)[min(base + j * kT + tid, nw128 - 1)];
    }
    // every slot of the round is loaded, index clamped (a slot past the end re-reads the last word and is not used)
    u32x4_t v[NS];
    uint64_t adr[NS];
#pragma unroll
    for (int j = 0; j < NS; ++j)
      adr[j] = reinterpret_cast<uint64_t>(in) + ((uint64_t)(uint32_t)min(base + j * kT + tid, nw128 - 1) << 4);
    // A round whose words have not all arrived is read again as a whole after a short sleep: one trip through memory per
    // attempt for the whole vector, however many producers are late (retrying word by word pays a trip per late word)
    for (int spins = 0;; ++spins) {
      ld_coh128_round(v, adr);
      bool late = false;
#pragma unroll
      for (int j = 0; j < NS; ++j) {
        if (base + j * kT >= nw128) break;
        if (base + j * kT + tid < nw128)
          late = late || (v[j].x >> 16) != tin || (v[j].y >> 16) != tin || (v[j].z >> 16) != tin || (v[j].w >> 16) != tin;
      }
      if (!__any(late ? 1 : 0)) break;
      if (spins >= limit || ((spins & 255) == 255 && ld_err(st) != 0)) { fail = fail || late; break; }
      __builtin_amdgcn_s_sleep(2);
    }
#pragma unroll
    for (int j = 0; j < NS; ++j) {
      if (base + j * kT >= nw128) break;
      const int q = base + j * kT + tid;
      if (q < nw128) {
        const uint32_t a0 = v[j].x & 0xffffu, a1 = v[j].y & 0xffffu, a2 = v[j].z & 0xffffu, a3 = v[j].w & 0xffffu;
        if (norm) {
          const float f0 = E::val(a0), f1 = E::val(a1), f2 = E::val(a2), f3 = E::val(a3);
          ss += (f0 * f0 + f1 * f1) + (f2 * f2 + f3 * f3);
          v[j].x = a0 | (a1 << 16);       // raw values; scaled once the sum is known
          v[j].y = a2 | (a3 << 16);
        } else {
          stage_store_wide<E>(xs, xsum, q, a0 | (a1 << 16), a2 | (a3 << 16), q4);
        }
      }
    }
    if (norm) {
      ss = wave_sum(ss);
      if ((tid & 63) == 0) red[tid >> 6] = ss;
      __syncthreads();
      float tot = 0.f;
#pragma unroll
      for (int i = 0; i < kT / 64; ++i) tot += red[i];
      const float rs = rsqrtf(tot / (float)in_len + eps);
#pragma unroll
      for (int j = 0; j < NS; ++j) {
        if (base + j * kT >= nw128) break;
        const int q = base + j * kT + tid;
        if (q < nw128) {
          const float f0 = E::lo(v[j].x), f1 = E::hi(v[j].x), f2 = E::lo(v[j].y), f3 = E::hi(v[j].y);
          stage_store_wide<E>(xs, xsum, q, E::pack2(E::lo(nwt[j].x) * E::rnd(f0 * rs), E::hi(nwt[j].x) * E::rnd(f1 * rs)),
                           E::pack2(E::lo(nwt[j].y) * E::rnd(f2 * rs), E::hi(nwt[j].y) * E::rnd(f3 * rs)), q4);
        }
      }
    }
  }
  return !fail;
}

// Staging for the composed form of a layer (FSVD_PF_STAGE2): `a` holds `na` fp32 sums in 64-bit tagged words (products
// with a hidden state that were completed, unrounded, by the previous phases), `b` the `nb` bf16 values of that hidden
// state itself.  One round of loads brings both; b goes to LDS as it is (at boff, for a phase that follows without a
// hand-off) and gives rs = rsqrt(mean(b^2) + eps); a goes to LDS as bf16(a * rs) at 0: the RMSNorm of the hidden state
// applied as a scalar behind the product (its weight vector is folded into the matrix).
template <class E, int NS>
__device__ __forceinline__ bool stage_pair(const void* a, int na, uint32_t ta, const void* b, int nb, uint32_t tb, int boff, float eps,
                                           const fsvd_step_state* st, int limit, uint16_t* xs, float* red) {
  const int tid = threadIdx.x;
  const int npa = na >> 1, npb = nb >> 2;          // 16-byte pieces: two 64-bit words of a, four 32-bit words of b
  const int sa = (npa + kT - 1) / kT;              // slots of a round that belong to a; the others to b (sa + sb <= NS, host-checked)
  u32x4_t v[NS];
  uint64_t adr[NS];
#pragma unroll
  for (int j = 0; j < NS; ++j) {                   // every slot is loaded, index clamped
    const bool isa = j < sa;
    const int q = (isa ? j : j - sa) * kT + tid;
    adr[j] = reinterpret_cast<uint64_t>(isa ? a : b) + ((uint64_t)(uint32_t)min(q, (isa ? npa : npb) - 1) << 4);
  }
  bool fail = false;
  for (int spins = 0;; ++spins) {
    ld_coh128_round(v, adr);
    bool late = false;
#pragma unroll
    for (int j = 0; j < NS; ++j) {
      const bool isa = j < sa;
      const int q = (isa ? j : j - sa) * kT + tid;
      if (isa) {
        if (q < npa) late = late || v[j].y != ta || v[j].w != ta;
      } else if (q < npb) {
        late = late || (v[j].x >> 16) != tb || (v[j].y >> 16) != tb || (v[j].z >> 16) != tb || (v[j].w >> 16) != tb;
      }
    }
    if (!__any(late ? 1 : 0)) break;
    if (spins >= limit || ((spins & 255) == 255 && ld_err(st) != 0)) { fail = late; break; }
    __builtin_amdgcn_s_sleep(2);
  }
  float ss = 0.f;
  uint2* xb = reinterpret_cast<uint2*>(xs + boff);
#pragma unroll
  for (int j = 0; j < NS; ++j) {
    const int q = (j - sa) * kT + tid;
    if (j >= sa && q < npb) {
      const uint32_t a0 = v[j].x & 0xffffu, a1 = v[j].y & 0xffffu, a2 = v[j].z & 0xffffu, a3 = v[j].w & 0xffffu;
      const float f0 = E::val(a0), f1 = E::val(a1), f2 = E::val(a2), f3 = E::val(a3);
      ss += (f0 * f0 + f1 * f1) + (f2 * f2 + f3 * f3);
      xb[q] = make_uint2(a0 | (a1 << 16), a2 | (a3 << 16));
    }
  }
  ss = wave_sum(ss);
  if ((tid & 63) == 0) red[tid >> 6] = ss;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int i = 0; i < kT / 64; ++i) tot += red[i];
  const float rs = rsqrtf(tot / (float)nb + eps);
  uint32_t* xa = reinterpret_cast<uint32_t*>(xs);
#pragma unroll
  for (int j = 0; j < NS; ++j) {
    const int q = j * kT + tid;
    if (j < sa && q < npa) xa[q] = E::pack2(__uint_as_float(v[j].x) * rs, __uint_as_float(v[j].z) * rs);
  }
  return !fail;
}

// ---------------------------------------------------------------------------------------------
// attention phase: this workgroup = (head h, key split s) over the keys already cached; the split that
// owns the current token also rotates and appends the new k / v
// ---------------------------------------------------------------------------------------------
struct AttnWork {
  int h, hk, s, k0, k1, newtok, nsplit, H, Hk;
  const uint16_t* kbase; const uint16_t* vbase;
  int64_t sc_s;
};
__device__ __forceinline__ void attn_setup(uint32_t dv, int w, int pos, AttnWork& a) {
  a.nsplit = DF_I(dv, nsplit);
  a.H = DF_I(dv, H);
  a.Hk = DF_I(dv, Hk);
  const int S = DF_I(dv, S);
  a.h = w / a.nsplit;
  a.s = w - a.h * a.nsplit;
  a.hk = a.h / (a.H / a.Hk);
  const int n_old = min(max(pos, 0), S);
  int per = (n_old + a.nsplit - 1) / a.nsplit;
  per = (per + kSlots - 1) / kSlots * kSlots;
  a.k0 = min(a.s * per, n_old);
  a.k1 = min(n_old, a.k0 + per);
  a.newtok = (a.s == a.nsplit - 1);
  const int part = threadIdx.x & 15;
  const int64_t sc_h = (int64_t)desc_u64(dv, FSVD_DW(sc_h));
  a.sc_s = (int64_t)desc_u64(dv, FSVD_DW(sc_s));
  a.kbase = static_cast<const uint16_t*>(DF_P(dv, k_cache)) + (int64_t)a.hk * sc_h + part * 8;
  a.vbase = static_cast<const uint16_t*>(DF_P(dv, v_cache)) + (int64_t)a.hk * sc_h + part * 8;
}
__device__ __forceinline__ void attn_window_addr(const AttnWork& a, int c0, uint64_t (&addr)[kU]) {
  const int slot = threadIdx.x >> 4;
#pragma unroll
  for (int u = 0; u < kUA; ++u) {
    const int key = max(0, min(c0 + u * kSlots + slot, a.k1 - 1));
    addr[u] = reinterpret_cast<uint64_t>(a.kbase + (int64_t)key * a.sc_s);
    addr[kUA + u] = reinterpret_cast<uint64_t>(a.vbase + (int64_t)key * a.sc_s);
  }
}
__device__ __forceinline__ void attn_issue(const AttnWork& a, int c0, u32x4_t (&R)[kU]) {
  uint64_t addr[kU];
  attn_window_addr(a, c0, addr);
#pragma unroll
  for (int u = 0; u < kU; ++u) R[u] = ld_stream(addr[u], 0);
}
template <class E>
__device__ __forceinline__ void softmax_step(float sc, const u32x4_t& v, float& m, float& l, float (&acc)[8]) {
  const float m_new = fmaxf(m, sc);
  const float alpha = (m == -INFINITY) ? 0.f : __expf(m - m_new);
  const float p = __expf(sc - m_new);
  acc[0] = acc[0] * alpha + p * E::lo(v.x); acc[1] = acc[1] * alpha + p * E::hi(v.x);
  acc[2] = acc[2] * alpha + p * E::lo(v.y); acc[3] = acc[3] * alpha + p * E::hi(v.y);
  acc[4] = acc[4] * alpha + p * E::lo(v.z); acc[5] = acc[5] * alpha + p * E::hi(v.z);
  acc[6] = acc[6] * alpha + p * E::lo(v.w); acc[7] = acc[7] * alpha + p * E::hi(v.w);
  l = l * alpha + p;
  m = m_new;
}

// Addresses of the first window of the phase described by dv.  The loads themselves are issued at ONE
// place in the kernel, straight into the window registers: a second issue site would make the compiler
// merge two register sets, which it does by waiting for every load and copying.
template <bool Q4, int QB>
__device__ __forceinline__ void window_addresses(uint32_t dv, int w, int pos, uint64_t dummy, uint64_t (&addr)[kU], uint64_t (&addr_sz)[kSzLoads]) {
  const int type = DF_I(dv, type);
#pragma unroll
  for (int u = 0; u < kU; ++u) addr[u] = dummy;
#pragma unroll
  for (int j = 0; j < kSzLoads; ++j) addr_sz[j] = dummy;
  if (type == FSVD_PH_GEMV) {
    GemvCtx c;
    gemv_ctx<Q4, QB>(dv, w, c);
    if (c.nmat == 1) gemv_window_addr<1>(c, addr);
    else gemv_window_addr<2>(c, addr);
    if (Q4 && c.q4) gemv_sz_table_addr(c, addr_sz);
  } else if (type == FSVD_PH_ATTN) {
    AttnWork aw;
    attn_setup(dv, w, pos, aw);
    attn_window_addr(aw, aw.k0, addr);
  }
}

__device__ __forceinline__ void raise_error(fsvd_step_state* st, int p, int w) {
  if (threadIdx.x == 0) {
    __hip_atomic_store(&st->err, p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    st->err_wg = w;
  }
}

// TRACE: workgroups 0, stride, 2*stride, ... record wall-clock ticks (100 MHz) per phase:
// [0] phase entered, [1] input staged, [2] weights consumed, [3] epilogue done
// Q4: the list may hold int4 GEMV phases; the build without them keeps the 16-bit walk free of their code
// CX: the list may hold the phases of the composed form (FSVD_PF_* flags, fp32 rows); likewise a build of its own
template <bool TRACE, bool Q4, bool CX, int DT>
__global__ __launch_bounds__(kT) void decode_step_kernel(const fsvd_phase* __restrict__ phases, int nph, fsvd_step_state* st,
                                                         unsigned long long* trace, int trace_stride) {
  typedef E16<DT> E;
  constexpr int QB = DT ? FSVD_WBITS_Q4_FP16 : 4;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  uint16_t* xs = reinterpret_cast<uint16_t*>(smem_raw);
  float* cp = reinterpret_cast<float*>(smem_raw + (size_t)kMaxIn * 2);
  float* red = cp + kMaxChunks;            // 32 floats
  int* ired = reinterpret_cast<int*>(red + 32);
  float* xsum = reinterpret_cast<float*>(smem_raw + (size_t)kMaxIn * 2 + (size_t)kMaxChunks * 4 + 256);   // [kMaxPieces]
  uint32_t* sztab = reinterpret_cast<uint32_t*>(xsum + kMaxPieces);                                        // [kMaxSz]

  const int tid = threadIdx.x, w = blockIdx.x, nwg = gridDim.x;
  if (st->err != 0) return;
  const int epoch = st->epoch, pos = st->pos;
  const long long token = st->token;
  const int limit = st->spin_limit > 0 ? st->spin_limit : kSpinLimit;

  u32x4_t R[kU];
  uint32_t SZ[kSzLoads];                   // int4 phases: this lane's words of the slab's scale | zero table, on their way to LDS
  uint32_t dvA = desc_fetch(phases, 0, nph), dvB = dvA;   // descriptors of phase p and p+1

  // Iteration p: finish phase p (its first weights were requested one iteration earlier), publish its
  // outputs, request the first weights of phase p+1.  (A leading phase, FSVD_PF_LEAD, only streams: its sums wait in
  // the partial buffer for the epilogue of the phase behind it.)
  int lead_chunks = 0;                     // chunk partials a leading phase left for this iteration's epilogue
  uint32_t dvL = dvA;                      // and its descriptor
  for (int p = -1; p < nph; ++p) {
    const uint32_t dvC = desc_fetch(phases, p + 2, nph);   // needed one iteration from now
    const uint32_t dv = dvA;
    const int pm = p;
    int type = p < 0 ? -1 : DF_I(dv, type);
    unsigned long long* tr = nullptr;
    if (TRACE && p >= 0 && tid == 0 && (w % trace_stride) == 0) {
      tr = trace + ((size_t)(w / trace_stride) * nph + p) * 4;
      tr[0] = wall_clock64();
    }
    GemvCtx gc;
    float* cpm = cp + lead_chunks;         // chunk partials of this phase (behind those of a leading phase)
    AttnWork aw;
    uint32_t resid = 0;
    int rows0 = 0x7fffffff;                // GEMV: first row of the fp32 group
    float addend = 0.f;                    // GEMV: this lane group's fp32 addend (second row group)
    // addresses of the next phase's first window, worked out now (behind the wait for this phase's input) so that the
    // request after publication is nothing but the loads
    uint64_t nxt[kU], nxt_sz[kSzLoads];
    window_addresses<Q4, QB>(dvB, w, pos, reinterpret_cast<uint64_t>(phases), nxt, nxt_sz);

    // ------------------------------------------------------------------ stage + stream
    if (CX && type == FSVD_PH_GEMV && (DF_I(dv, flags) & FSVD_PF_LEAD) != 0) {
      gemv_ctx<false, 4>(dv, w, gc);
      // the epilogue of the previous phase may still be reading the partial buffer in another wave (its LDS reads are
      // complete by the time that wave's stores have been issued, i.e. before it arrives here)
      __builtin_amdgcn_s_barrier();
      lead_stream<E>(gc, desc_u32(dv, FSVD_DW(m_kp)), R, xs + gc.xoff, cp);
      lead_chunks = gc.pps >> 4;
      dvL = dv;
      if (TRACE && tr) tr[1] = tr[0];      // nothing staged
      type = -2;                           // no staging, no epilogue: on to the window request
    }
    if (type == FSVD_PH_GEMV) {
      gemv_ctx<Q4, QB>(dv, w, gc);
      const int epi = DF_I(dv, epilogue);
      const int flags = CX ? DF_I(dv, flags) : 0;
      if (CX) rows0 = (flags & FSVD_PF_SPLIT) ? DF_I(dv, rows0) : (epi == FSVD_EP_F32 ? 0 : 0x7fffffff);
      const int myrow = gc.r0 + (tid >> 3);          // the row whose epilogue this lane group runs (one pass: host-checked)
      if (epi == FSVD_EP_RESID && (tid >> 3) < gc.srows && myrow < rows0) resid = ld_coh32(DF_P(dv, aux0), myrow);
      // fp32 addend of a row of the second group: requested now, its tag checked behind the staging (it was published
      // several hand-offs ago, but by another workgroup and to no reader before this one: nothing else proves it visible)
      const void* aux2p = CX && desc_u64(dv, FSVD_DW(aux2)) != 0 ? DF_P(dv, aux2) : nullptr;
      const bool want2 = aux2p != nullptr && (tid >> 3) < gc.srows && myrow >= rows0;
      uint64_t a2w = 0;
      if (want2) a2w = ld_coh64(aux2p, myrow - rows0);
      const int gH = DF_I(dv, H);                 // > 0: rows are q | k | v groups with their own inputs
      const int in_len = (gH > 0 ? 3 : (gc.xk ? gc.nmat : 1)) * gc.K;
      const uint32_t tin = DF_TAG16(dv, in, epoch);
      const uint32_t* nw = static_cast<const uint32_t*>(DF_P(dv, norm_w));
      bool ok = true;
      const void* inp = DF_P(dv, in);
      if (flags & FSVD_PF_NOWAIT) {
        // the previous phase of this workgroup staged the input; its epilogue may still be reading the partial buffer
      } else if (flags & FSVD_PF_STAGE2) {
        const int n2 = DF_I(dv, in2_len);
        const int slots = ((in_len >> 1) + kT - 1) / kT + ((n2 >> 2) + kT - 1) / kT;
        if (slots <= 5)
          ok = stage_pair<E, 5>(inp, in_len, DF_TAG32(dv, in, epoch), DF_P(dv, in2), n2, DF_TAG16(dv, in2, epoch), DF_I(dv, in2_off),
                             DF_F(dv, fparam), st, limit, xs, red);
        else
          ok = stage_pair<E, 8>(inp, in_len, DF_TAG32(dv, in, epoch), DF_P(dv, in2), n2, DF_TAG16(dv, in2, epoch), DF_I(dv, in2_off),
                             DF_F(dv, fparam), st, limit, xs, red);
      } else if (in_len <= 2 * kT * 4) {
        ok = stage_input_wide<E, 2>(inp, in_len, tin, nw, DF_F(dv, fparam), st, limit, xs, red, Q4 && gc.q4, xsum);
      } else {
        ok = stage_input_wide<E, 8>(inp, in_len, tin, nw, DF_F(dv, fparam), st, limit, xs, red, Q4 && gc.q4, xsum);
      }
      // Every load of the staging code has been consumed by now (and the window, requested before the polls, has landed
      // with them: loads complete in order).  The compiler's bookkeeping cannot see that for loads issued under a
      // condition; without this explicit (and free) wait it protects the registers they used with full waits in the
      // middle of the weight stream's batches, which halves the loads in flight there.
      __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0), no wait on the other counters
      if (want2) {
        const uint32_t t2 = DF_TAG32(dv, aux2, epoch);
        uint32_t pay = (uint32_t)a2w;
        if ((uint32_t)(a2w >> 32) != t2 && !poll_w64(aux2p, myrow - rows0, t2, st, limit, pay)) ok = false;
        addend = __uint_as_float(pay);
      }
      if (Q4 && gc.q4) {   // the slab's scale | zero table came with the window, ahead of the polls; the barrier publishes it
#pragma unroll
        for (int j = 0; j < kSzLoads; ++j) sztab[j * kT + tid] = SZ[j];
      }
      // an int4 phase in a 16-bit build, or a phase of the composed form in a build without it, is an error too
      if (__syncthreads_or((ok && (Q4 || DF_I(dv, wbits) != QB) && (CX || (DF_I(dv, flags) == 0 && epi != FSVD_EP_F32))) ? 0 : 1)) {
        raise_error(st, pm, w);
        return;
      }
      if (TRACE && tr) tr[1] = wall_clock64();
      const uint32_t m_kp = desc_u32(dv, FSVD_DW(m_kp));
      if (Q4 && gc.q4) {
        if (gH > 0) {
          const int g1 = gH * DF_I(dv, Dh), g2 = (gH + DF_I(dv, Hk)) * DF_I(dv, Dh);
          gemv_stream_q4<E, 1, true>(gc, m_kp, g1, g2, R, sztab, xs, xsum, cp);
        } else if (gc.nmat == 1) {
          gemv_stream_q4<E, 1, false>(gc, m_kp, 0, 0, R, sztab, xs, xsum, cp);
        } else {
          gemv_stream_q4<E, 2, false>(gc, m_kp, 0, 0, R, sztab, xs, xsum, cp);
        }
      } else if (gH > 0) {
        const int g1 = gH * DF_I(dv, Dh), g2 = (gH + DF_I(dv, Hk)) * DF_I(dv, Dh);
        gemv_stream<E, 1, true>(gc, m_kp, g1, g2, R, xs + (CX ? gc.xoff : 0), cp);
      } else if (gc.nmat == 1) {
        gemv_stream<E, 1, false>(gc, m_kp, 0, 0, R, xs + (CX ? gc.xoff : 0), cpm);
      } else {
        gemv_stream<E, 2, false>(gc, m_kp, 0, 0, R, xs + (CX ? gc.xoff : 0), cp);
      }
      __syncthreads();
    } else if (type == FSVD_PH_ATTN) {
      // q of this head, rotated here (the projection phase publishes q, k, v un-rotated); the split that
      // owns the current token also rotates k, keeps k / v in LDS as its extra key and appends them to
      // the cache for later steps (one query head per kv head does the append)
      attn_setup(dv, w, pos, aw);
      const int Dh = 128, half = 64;
      const uint32_t tq = DF_TAG16(dv, in, epoch);
      const void* qkv = DF_P(dv, in);
      const uint16_t* cosT = static_cast<const uint16_t*>(DF_P(dv, cos));
      const uint16_t* sinT = static_cast<const uint16_t*>(DF_P(dv, sin));
      bool fail = false;
      const int role = tid >> 6;                 // wave 0: q pairs, wave 1: k pairs, wave 2: v pairs
      const int dd = tid & 63;
      if (role == 0 || (role <= 2 && aw.newtok)) {
        const int ebase = role == 0 ? aw.h * Dh : (role == 1 ? (aw.H + aw.hk) * Dh : (aw.H + aw.Hk + aw.hk) * Dh);
        float c = 1.f, sn = 0.f;
        if (role != 2 && cosT) {
          const int tp = min(max(pos, 0), DF_I(dv, rope_len) - 1);
          c = E::val(cosT[(int64_t)tp * half + dd]);
          sn = E::val(sinT[(int64_t)tp * half + dd]);
        }
        // the two halves of a rotation pair in one trip through memory: both loads, then both tags
        uint32_t b0, b1;
        for (int spins = 0;;) {
          const uint32_t v0 = ld_coh32(qkv, ebase + dd), v1 = ld_coh32(qkv, ebase + dd + half);
          b0 = v0 & 0xffffu;
          b1 = v1 & 0xffffu;
          if ((v0 >> 16) == tq && (v1 >> 16) == tq) break;
          if (++spins > limit || ((spins & 1023) == 0 && ld_err(st) != 0)) { fail = true; break; }
        }
        float x0 = E::val(b0), x1 = E::val(b1);
        if (role != 2 && cosT) {
          // eager bf16 arithmetic: one rounding per multiply and per add
          const float r0 = E::rnd(E::rnd(x0 * c) - E::rnd(x1 * sn));
          const float r1 = E::rnd(E::rnd(x1 * c) + E::rnd(x0 * sn));
          x0 = r0; x1 = r1;
        }
        const uint16_t o0 = (uint16_t)E::bits(x0), o1 = (uint16_t)E::bits(x1);
        xs[role * Dh + dd] = o0;
        xs[role * Dh + dd + half] = o1;
        if (role != 0 && aw.h == aw.hk * (aw.H / aw.Hk) && pos >= 0 && pos < DF_I(dv, S)) {
          uint16_t* cb = static_cast<uint16_t*>(role == 1 ? DF_P(dv, k_cache) : DF_P(dv, v_cache)) + (int64_t)pos * aw.sc_s +
                         (int64_t)aw.hk * (int64_t)desc_u64(dv, FSVD_DW(sc_h)) + dd;
          cb[0] = o0;
          cb[half] = o1;
        }
      }
      if (__syncthreads_or(fail ? 1 : 0)) { raise_error(st, pm, w); return; }
      if (TRACE && tr) tr[1] = wall_clock64();
      const float scale = DF_F(dv, fparam);
      const int part = tid & 15, slot = tid >> 4;
      const u32x4_t qv = *reinterpret_cast<const u32x4_t*>(xs + part * 8);
      float m_run = -INFINITY, l_run = 0.f;
      float acc[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = 0.f;
      for (int c0 = aw.k0; c0 < aw.k1; c0 += kSlots * kUA) {
        if (c0 != aw.k0) attn_issue(aw, c0, R);
#pragma unroll
        for (int u = 0; u < kUA; ++u) {
          const float sc = row16_sum(E::dot8(R[u], qv, 0.f)) * scale;
          if (c0 + u * kSlots + slot < aw.k1) softmax_step<E>(sc, R[kUA + u], m_run, l_run, acc);
        }
      }
      if (aw.newtok && slot == 0) {
        const u32x4_t kn = *reinterpret_cast<const u32x4_t*>(xs + Dh + part * 8);
        const u32x4_t vn = *reinterpret_cast<const u32x4_t*>(xs + 2 * Dh + part * 8);
        const float sc = row16_sum(E::dot8(kn, qv, 0.f)) * scale;
        softmax_step<E>(sc, vn, m_run, l_run, acc);
      }
      // park the key slots: cp[slot][Dh + 2]
      float* sl = cp + slot * (Dh + 2);
#pragma unroll
      for (int i = 0; i < 8; ++i) sl[part * 8 + i] = acc[i];
      if (part == 0) { sl[Dh] = m_run; sl[Dh + 1] = l_run; }
      __syncthreads();
    }
    if (TRACE && tr) tr[2] = wall_clock64();

    // ------------------------------------------------------------------ publish (GEMV, attention)
    if (type == FSVD_PH_GEMV) {
      const int epi = DF_I(dv, epilogue);
      const int cpr = gc.q4 ? gc.kp >> 3 : gc.kp >> 4;   // chunks per row: 256 columns (int4) or 128
      const uint32_t tout = DF_TAG16(dv, out0, epoch);
      void* out = DF_P(dv, out0);
      const int grp = tid >> 3;
      const bool lead8 = (tid & 7) == 0;
      const int npass = (gc.srows + kT / 8 - 1) / (kT / 8);
      if (epi == FSVD_EP_LOGITS) {
        float best = -INFINITY;
        int best_i = 0x7fffffff;
        uint16_t* logits = static_cast<uint16_t*>(DF_P(dv, plain_out));
        for (int ps = 0; ps < npass; ++ps) {
          const int t = min(ps * (kT / 8) + grp, gc.srows - 1);
          const float v = E::rnd(row_sum8(cp, t, cpr));
          if (lead8 && ps * (kT / 8) + grp < gc.srows) {
            logits[gc.r0 + t] = (uint16_t)E::bits(v);
            if (v > best) { best = v; best_i = gc.r0 + t; }
          }
        }
        // fold (value, index) over the workgroup; ties go to the lower index
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
          const float ov = __shfl_xor(best, off);
          const int oi = __shfl_xor(best_i, off);
          if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
        }
        if ((tid & 63) == 0) { red[tid >> 6] = best; ired[tid >> 6] = best_i; }
        __syncthreads();
        if (tid == 0) {
          for (int i = 1; i < kT / 64; ++i)
            if (red[i] > best || (red[i] == best && ired[i] < best_i)) { best = red[i]; best_i = ired[i]; }
          const uint64_t word = ((uint64_t)((tout << 16) | E::bits(best)) << 32) | (uint32_t)best_i;
          __hip_atomic_store(static_cast<uint64_t*>(out) + w, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();   // `red` is reused by the argmax phase
      } else if ((tid >> 6) * 8 < gc.srows) {   // waves whose lane groups own no row skip the epilogue
        const int mode = DF_I(dv, mode);
        for (int ps = 0; ps < npass; ++ps) {
          const int t = min(ps * (kT / 8) + grp, gc.srows - 1);
          const bool live = lead8 && ps * (kT / 8) + grp < gc.srows;
          float v;
          if (CX && gc.r0 + t >= rows0) {      // fp32 row group: the unrounded sum (+ the part of it an earlier phase left)
            v = row_sum8(cpm, t, cpr) + addend;
            if (live) st_tag64(DF_P(dv, out1), gc.r0 + t - rows0, DF_TAG32(dv, out1, epoch), __float_as_uint(v));
            continue;
          }
          if (epi == FSVD_EP_SWIGLU) {
            float gv = row_sum8(cp, t, cpr), uv = row_sum8(cp, gc.srows + t, cpr);
            if (mode == 0) {
              gv = E::rnd(gv);
              uv = E::rnd(uv);
              v = E::rnd(E::rnd(silu_f32(gv)) * uv);
            } else {
              v = E::rnd((gv * (1.0f / (1.0f + expf(-gv)))) * uv);
            }
          } else {
            v = E::rnd(row_sum8(cpm, t, cpr));
            if (epi == FSVD_EP_RESID) v = E::rnd(E::val(resid & 0xffffu) + v);
          }
          if (live) st_tag16(out, gc.r0 + t, tout, E::bits(v));
        }
      }
      if (CX && lead_chunks != 0) {
        // the rows of the leading phase in front of this one: unrounded sums, taken by the lane groups from the top of the
        // workgroup down while those from the bottom up run this phase's epilogue
        GemvCtx fc;
        gemv_ctx<false, 4>(dvL, w, fc);
        const int t = kT / 8 - 1 - grp;
        if (t < fc.srows) {
          const float v = row_sum8(cp, t, fc.kp >> 4);
          if (lead8) st_tag64(DF_P(dvL, out1), fc.r0 + t, DF_TAG32(dvL, out1, epoch), __float_as_uint(v));
        }
        lead_chunks = 0;
      }
      // no barrier here: the next phase writes cp only after its staging barrier (a leading phase: after a barrier of
      // its own), which every wave reaches after this epilogue
    } else if (type == FSVD_PH_ATTN) {
      // fold the key slots and publish this split's (acc, m, l)
      const int Dh = 128;
      float* wts = cp + kSlots * (Dh + 2);     // kSlots weights, then the maximum
      if (tid < 64) {
        const float mj = tid < kSlots ? cp[tid * (Dh + 2) + Dh] : -INFINITY;
        const float M0 = wave_max(mj);
        if (tid < kSlots) wts[tid] = (mj == -INFINITY) ? 0.f : __expf(mj - M0);
        if (tid == 0) wts[kSlots] = M0;
      }
      __syncthreads();
      if (tid < Dh + 2) {
        const float M = wts[kSlots];
        float o = M;
        if (tid != Dh) {
          const int col = tid < Dh ? tid : Dh + 1;
          o = 0.f;
#pragma unroll 8
          for (int j = 0; j < kSlots; ++j) o += wts[j] * cp[j * (Dh + 2) + col];
        }
        st_tag64(DF_P(dv, out0), (aw.h * aw.nsplit + aw.s) * (Dh + 2) + tid, DF_TAG32(dv, out0, epoch), __float_as_uint(o));
      }
      __syncthreads();   // the merge phase reuses cp without a barrier of its own in front
    }

    // ------------------------------------------------------------------ first window of the next phase
    // (the only place window loads are issued outside the streaming loops; phases without weights read a
    // dummy line so that the registers are always written here)
#pragma unroll
    for (int u = 0; u < kU; ++u) R[u] = ld_stream(nxt[u], 0);
    if (Q4) {
#pragma unroll
      for (int j = 0; j < kSzLoads; ++j) SZ[j] = ld_stream32(nxt_sz[j]);
    }

    // ------------------------------------------------------------------ phases that poll after the request
    if (type == FSVD_PH_EMBED) {
      const int q = DF_I(dv, share_q), r = DF_I(dv, share_r), N = DF_I(dv, N);
      const int n0 = w * q + min(w, r), n1 = n0 + q + (w < r ? 1 : 0);
      // K > 0 is the number of rows of the table: a token outside it (a caller's mistake, or the index the argmax
      // leaves when no logit compares) must not become an address; row 0 is read instead and the step reports it
      const int V = DF_I(dv, K);
      long long tk = token;
      if (V > 0 && (tk < 0 || tk >= V)) { tk = 0; raise_error(st, pm, w); }
      const uint16_t* row = static_cast<const uint16_t*>(DF_P(dv, W)) + tk * (int64_t)N;
      const uint32_t tg = DF_TAG16(dv, out0, epoch);
      void* out = DF_P(dv, out0);
      for (int n = n0 + tid; n < n1; n += kT) st_tag16(out, n, tg, row[n]);
    } else if (type == FSVD_PH_MERGE) {
      // merge the key splits: this workgroup owns `cnt` consecutive output elements of one head; one
      // lane polls one word (cnt accumulators + m + l for every split), so all polls are in flight at once
      const int Dh = 128, dsh = 7;
      const int cnt = DF_I(dv, share_q);         // H * Dh / workgroups
      const int nsplit = DF_I(dv, nsplit);
      const int o0 = w * cnt;
      const int head = o0 >> dsh, dim0 = o0 - (head << dsh);
      const uint32_t tin = DF_TAG32(dv, in, epoch), tout = DF_TAG16(dv, out0, epoch);
      const void* in = DF_P(dv, in);
      const int per = cnt + 2, items = nsplit * per;
      bool fail = false;
      for (int it = tid; it < items; it += kT) {
        const int sp = it / per, j = it - sp * per;
        const int col = j < cnt ? dim0 + j : Dh + (j - cnt);
        uint32_t payload;
        if (!poll_w64(in, (head * nsplit + sp) * (Dh + 2) + col, tin, st, limit, payload)) fail = true;
        cp[it] = __uint_as_float(payload);
      }
      if (__syncthreads_or(fail ? 1 : 0)) { raise_error(st, pm, w); return; }
      if (tid < cnt) {
        float M = -INFINITY, num = 0.f, den = 0.f;
        for (int sp = 0; sp < nsplit; ++sp) M = fmaxf(M, cp[sp * per + cnt]);
        for (int sp = 0; sp < nsplit; ++sp) {
          const float mi = cp[sp * per + cnt];
          const float wi = (mi == -INFINITY) ? 0.f : __expf(mi - M);
          num += wi * cp[sp * per + tid];
          den += wi * cp[sp * per + cnt + 1];
        }
        st_tag16(DF_P(dv, out0), o0 + tid, tout, E::bits(den > 0.f ? num / den : 0.f));
      }
    } else if (type == FSVD_PH_ARGMAX) {
      // greedy token, state advance
      if (w == 0) {
        const uint32_t tin = DF_TAG16(dv, in, epoch);
        const void* in = DF_P(dv, in);
        float best = -INFINITY;
        int best_i = 0x7fffffff;
        bool fail = false;
        for (int t = tid; t < nwg; t += kT) {
          int spins = 0;
          for (;;) {
            const uint64_t v = ld_coh64(in, t);
            if ((uint32_t)(v >> 48) == tin) {
              const float val = E::val((uint32_t)(v >> 32) & 0xffffu);
              const int idx = (int)(uint32_t)v;
              if (val > best || (val == best && idx < best_i)) { best = val; best_i = idx; }
              break;
            }
            if (++spins > limit || ((spins & 1023) == 0 && ld_err(st) != 0)) { fail = true; break; }
          }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
          const float ov = __shfl_xor(best, off);
          const int oi = __shfl_xor(best_i, off);
          if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
        }
        if ((tid & 63) == 0) { red[tid >> 6] = best; ired[tid >> 6] = best_i; }
        if (__syncthreads_or(fail ? 1 : 0)) { raise_error(st, pm, w); return; }
        if (tid == 0) {
          for (int i = 1; i < kT / 64; ++i)
            if (red[i] > best || (red[i] == best && ired[i] < best_i)) { best = red[i]; best_i = ired[i]; }
          // no logit compared greater than -inf (all NaN): there is no greedy token; token 0 stands in and the step says so
          if (best_i == 0x7fffffff) {
            best_i = 0;
            __hip_atomic_store(&st->err, pm + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            st->err_wg = w;
          }
          long long* log = static_cast<long long*>(DF_P(dv, plain_out));
          if (log) log[st->step] = best_i;
          st->token = best_i;
          st->pos = pos + 1;
          st->step = st->step + 1;
        }
      }
    }
    if (TRACE && tr) tr[3] = wall_clock64();
    if (p >= 0) dvA = dvB;   // iteration -1 already holds descriptor 0 in both
    dvB = dvC;
  }
  // Every workgroup read the state before it produced anything, and workgroup 0 cannot get here before
  // it has consumed data from all the others, so bumping the epoch now cannot be seen by this launch.
  if (w == 0 && tid == 0) st->epoch = epoch + 1;
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
static int g_step_wgs = 0;

// One workgroup per compute unit, all of them resident at once: a workgroup that waits for a hand-off spins, so a
// workgroup that is still waiting for a free compute unit would never get one.  The grid is therefore refused unless the
// runtime's own occupancy calculation places at least one workgroup of every instantiation on a compute unit (registers,
// LDS, waves); what the calculation cannot see - other kernels holding compute units while a step runs - is the
// caller's to avoid: nothing else may execute on the device during a step (a starved step ends by its spin limit with
// the error flag set, it does not hang).
int decode_step_workgroups() {
  if (g_step_wgs > 0) return g_step_wgs;
  int dev = 0;
  hipDeviceProp_t prop;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) {
    set_last_error("fsvd_decode_step: cannot query the device");
    return 0;
  }
  const void* fns[12] = {reinterpret_cast<const void*>(decode_step_kernel<false, false, false, 0>), reinterpret_cast<const void*>(decode_step_kernel<true, false, false, 0>),
                         reinterpret_cast<const void*>(decode_step_kernel<false, true, false, 0>), reinterpret_cast<const void*>(decode_step_kernel<true, true, false, 0>),
                         reinterpret_cast<const void*>(decode_step_kernel<false, false, true, 0>), reinterpret_cast<const void*>(decode_step_kernel<true, false, true, 0>),
                         reinterpret_cast<const void*>(decode_step_kernel<false, false, false, 1>), reinterpret_cast<const void*>(decode_step_kernel<true, false, false, 1>),
                         reinterpret_cast<const void*>(decode_step_kernel<false, false, true, 1>), reinterpret_cast<const void*>(decode_step_kernel<true, false, true, 1>),
                         reinterpret_cast<const void*>(decode_step_kernel<false, true, false, 1>), reinterpret_cast<const void*>(decode_step_kernel<true, true, false, 1>)};
  for (const void* fn : fns) {
    if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kSmemBytes) != hipSuccess) {
      set_last_error("fsvd_decode_step: the device refuses %zu bytes of dynamic LDS per workgroup", kSmemBytes);
      return 0;
    }
    int resident = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&resident, fn, kT, kSmemBytes) != hipSuccess || resident < 1) {
      set_last_error("fsvd_decode_step: a workgroup of the step kernel (%d threads, %zu bytes of LDS) does not fit a compute unit of "
                     "this device, so its grid of one workgroup per compute unit cannot be co-resident", kT, kSmemBytes);
      (void)hipGetLastError();
      return 0;
    }
  }
  g_step_wgs = prop.multiProcessorCount;
  return g_step_wgs;
}

int prepare_decode_step(fsvd_phase* ph, int nph, int nwg) {
  for (int p = 0; p < nph; ++p) {
    fsvd_phase& d = ph[p];
    int items = 0;
    if (d.type == FSVD_PH_EMBED || d.type == FSVD_PH_GEMV) items = d.N;
    else if (d.type == FSVD_PH_MERGE) items = d.H * d.Dh;
    d.share_q = items / nwg;
    d.share_r = items % nwg;
    d.m_kp = 0;
    d.dk = 0;
    const int pc = is_q4_bits(d.wbits) ? 32 : 8;   // columns per 16-byte piece
    if (d.type == FSVD_PH_GEMV && d.K >= pc) {
      d.m_kp = 0xffffffffu / (uint32_t)(d.K / pc) + 1u;
      d.dk = kT % (d.K / pc);
    }
  }
  return kOk;
}

static int bad(const char* what, int p) {
  set_last_error("fsvd_decode_step: phase %d: %s", p, what);
  return kErrBadShape;
}

// staged elements of a GEMV phase's own input
static int gemv_in_len(const fsvd_phase& d) { return (d.H > 0 ? 3 : (d.shared_in ? 1 : d.nmat)) * d.K; }

int validate_decode_step(const fsvd_phase* ph, int nph, int nwg) {
  if (nph < 2) return bad("a step needs at least two phases", 0);
  {
    bool any_q4 = false, any_cx = false, any_f16 = false, any_b16 = false;
    for (int p = 0; p < nph; ++p) {
      if (ph[p].type != FSVD_PH_GEMV) continue;
      any_q4 = any_q4 || is_q4_bits(ph[p].wbits);
      any_f16 = any_f16 || ph[p].wbits == FSVD_WBITS_FP16 || ph[p].wbits == FSVD_WBITS_Q4_FP16;
      any_b16 = any_b16 || ph[p].wbits == 0 || ph[p].wbits == 16 || ph[p].wbits == 4;
      any_cx = any_cx || ph[p].flags != 0 || ph[p].epilogue == FSVD_EP_F32;
    }
    if (any_q4 && any_cx) return bad("a list holds int4 phases or phases of the composed form, not both (they run on different builds of the kernel)", 0);
    // the element type belongs to the step: its vectors, tables and caches are all of one 16-bit type
    if (any_f16 && any_b16) return bad("a list is float16 in every GEMV phase (FSVD_WBITS_FP16, FSVD_WBITS_Q4_FP16) or in none", 0);
  }

  // Every tagged buffer with the phase that wrote it last.  `full`: every workgroup wrote part of it in that phase (a
  // consumer that has polled all of it knows that every workgroup is through that phase); `half`: it is one of the two
  // outputs of a phase with two row groups, which cover the workgroups only together.
  struct Seen { const void* ptr; int last_write; fsvd_tagbuf tb; bool full, half; };
  std::vector<Seen> seen;
  auto find = [&](const void* ptr) -> Seen* {
    for (auto& s : seen)
      if (s.ptr == ptr) return &s;
    return nullptr;
  };
  auto reads = [&](const fsvd_phase& d, const void* o) -> bool {
    if (!o) return false;
    if (d.type == FSVD_PH_GEMV) {
      if (!(d.flags & FSVD_PF_NOWAIT) && d.in.ptr == o) return true;
      if ((d.flags & FSVD_PF_STAGE2) && d.in2.ptr == o) return true;
      if (d.epilogue == FSVD_EP_RESID && d.aux0.ptr == o) return true;
      return d.aux2.ptr == o;
    }
    return d.in.ptr == o;
  };
  // the phase up to which every workgroup is known to have come once phase q has staged its input: the producer of a
  // fully polled vector that every workgroup helped to write (-1: none)
  std::vector<int> closes(nph, -1);
  for (int p = 0; p < nph; ++p) {
    const fsvd_phase& d = ph[p];
    {
      int items = 0;
      if (d.type == FSVD_PH_EMBED || d.type == FSVD_PH_GEMV) items = d.N;
      else if (d.type == FSVD_PH_MERGE) items = d.H * d.Dh;
      bool ok = d.share_q == items / nwg && d.share_r == items % nwg;
      const int pc = is_q4_bits(d.wbits) ? 32 : 8;
      if (d.type == FSVD_PH_GEMV && d.K >= pc)
        ok = ok && d.m_kp == 0xffffffffu / (uint32_t)(d.K / pc) + 1u && d.dk == kT % (d.K / pc);
      if (!ok) return bad("derived fields missing: call fsvd_decode_step_prepare", p);
    }
    bool out0_written = true, out1_written = false;
    switch (d.type) {
      case FSVD_PH_EMBED:
        if (p != 0) return bad("the embedding phase must come first", p);
        if (!d.W[0] || !d.out0.ptr || d.N < nwg) return bad("embedding phase needs W[0], out0 and N >= workgroups", p);
        break;
      case FSVD_PH_GEMV: {
        if (d.nmat < 1 || d.nmat > 2 || !d.W[0] || (d.nmat == 2 && !d.W[1])) return bad("GEMV needs 1 or 2 matrices", p);
        if (d.wbits != 0 && d.wbits != 16 && d.wbits != 4 && d.wbits != FSVD_WBITS_FP16 && d.wbits != FSVD_WBITS_Q4_FP16)
          return bad("wbits must be 0 / 16 (bf16), 4 (int4 under bf16), FSVD_WBITS_FP16 or FSVD_WBITS_Q4_FP16", p);
        const bool q4 = is_q4_bits(d.wbits);
        if (d.K <= 0 || d.K % (q4 ? 256 : 128) != 0) return bad(q4 ? "K must be a positive multiple of 256 for int4 weights" : "K must be a positive multiple of 128", p);
        if (q4) {
          if (!d.qsz[0] || (d.nmat == 2 && !d.qsz[1])) return bad("int4 GEMV needs the scale | zero words of every matrix", p);
          if (d.gshift < 0 || d.gshift > 20) return bad("bad group shift", p);
          if (d.ldg < (((d.K / 32) - 1) >> d.gshift) + 1) return bad("scale | zero rows shorter than the number of groups", p);
          if ((((int64_t)d.N + nwg - 1) / nwg) * d.ldg * d.nmat > kMaxSz) return bad("scale | zero table of a workgroup's rows does not fit its LDS buffer", p);
          for (int m = 0; m < d.nmat; ++m)
            if (reinterpret_cast<uintptr_t>(d.qsz[m]) & 3) return bad("scale | zero words must be 4-byte aligned", p);
        }
        if (d.N < nwg) return bad("fewer rows than workgroups", p);
        if (d.flags & ~(FSVD_PF_NOWAIT | FSVD_PF_STAGE2 | FSVD_PF_SPLIT | FSVD_PF_LEAD)) return bad("unknown flag", p);
        const bool nowait = d.flags & FSVD_PF_NOWAIT, stage2 = d.flags & FSVD_PF_STAGE2, split = d.flags & FSVD_PF_SPLIT;
        const bool leading = d.flags & FSVD_PF_LEAD;
        const bool f32rows = split || d.epilogue == FSVD_EP_F32;
        if ((d.flags != 0 || f32rows || d.in_off != 0) && q4) return bad("flags, fp32 rows and input offsets are for 16-bit weights", p);
        if (d.H > 0) {   // q | k | v row groups reading [Pq | Pk | Pv]
          if (d.nmat != 1 || d.epilogue != FSVD_EP_STORE || d.norm_w || split) return bad("grouped GEMV is a plain single-matrix store", p);
          if (d.Hk <= 0 || d.Dh <= 0 || d.N != (d.H + 2 * d.Hk) * d.Dh) return bad("grouped GEMV needs N = (H + 2*Hk) * Dh", p);
        }
        if (d.shared_in != 0 && (d.nmat != 2 || d.H > 0)) return bad("shared_in is for a pair of matrices over one input", p);
        const int n_in = gemv_in_len(d);
        if (d.in_off < 0 || d.in_off % 8 != 0 || (int64_t)d.in_off + n_in > kMaxIn) return bad("input does not fit the staging buffer", p);
        if (d.norm_w && n_in > kT * 12 * 2) return bad("normalised input too long for one staging round", p);
        if (nowait) {
          // the input is what the previous phase of the same workgroup left in its staging area
          if (stage2 || d.norm_w || d.aux2.ptr) return bad("a phase without a hand-off stages nothing and takes no addend", p);
          if (leading) {
            // streamed in front of the next phase: the input is what an earlier two-vector staging left at in_off, and
            // nothing since may have been staged over it
            if (d.epilogue != FSVD_EP_F32 || d.nmat != 1 || d.H > 0 || split)
              return bad("a leading phase is a single matrix whose rows leave as unrounded fp32 sums", p);
            if (d.N % nwg != 0 || d.N / nwg > kT / 8) return bad("a leading phase deals the same number of rows, at most kT/8, to every workgroup", p);
            if (((int64_t)(d.N / nwg) * (d.K / 8)) % (kT * kU) != 0) return bad("the slab of a leading phase must fill whole windows (rows per workgroup x K/8 a multiple of kT x kU)", p);
            if (p + 1 >= nph) return bad("a leading phase needs a phase behind it", p);
            const fsvd_phase& m = ph[p + 1];
            if (m.type != FSVD_PH_GEMV || m.nmat != 1 || m.H > 0 || m.flags != 0 || is_q4_bits(m.wbits) ||
                (m.epilogue != FSVD_EP_STORE && m.epilogue != FSVD_EP_RESID))
              return bad("the phase behind a leading phase must be a plain single-matrix bf16 GEMV that stores or adds a residual", p);
            if (d.in_off < gemv_in_len(m)) return bad("the staged input of a leading phase overlaps the input of the phase behind it", p);
            if ((int64_t)(d.N / nwg) * (d.K / 128) + (((int64_t)m.N + nwg - 1) / nwg) * (m.K / 128) > kMaxChunks)
              return bad("a leading phase and the phase behind it overflow the partial buffer", p);
            bool found = false;
            for (int q = p - 1; q >= 0 && !found; --q) {
              const fsvd_phase& e = ph[q];
              if (e.type == FSVD_PH_GEMV) {
                if ((e.flags & FSVD_PF_STAGE2) && e.in2_off == d.in_off && e.in2_len == n_in) { found = true; break; }
                if (e.flags & FSVD_PF_NOWAIT) continue;
                const bool hits2 = (e.flags & FSVD_PF_STAGE2) && e.in2_off < d.in_off + n_in && d.in_off < e.in2_off + e.in2_len;
                if (gemv_in_len(e) > d.in_off || hits2) return bad("the staged input of a leading phase was overwritten by a later staging", p);
              } else if (e.type == FSVD_PH_ATTN) {
                if (3 * e.Dh > d.in_off) return bad("the staged input of a leading phase was overwritten by an attention phase", p);
              } else if (e.type != FSVD_PH_MERGE) {
                break;
              }
            }
            if (!found) return bad("a leading phase must read a vector that an earlier two-vector staging left in place", p);
          } else {
          if (p == 0 || ph[p - 1].type != FSVD_PH_GEMV) return bad("a phase without a hand-off must follow a GEMV phase", p);
          const fsvd_phase& q = ph[p - 1];
          const bool from_in2 = (q.flags & FSVD_PF_STAGE2) && d.in_off == q.in2_off && n_in == q.in2_len;
          const bool same_in = d.in_off == q.in_off && n_in <= gemv_in_len(q) && !q.norm_w && !(q.flags & FSVD_PF_STAGE2);
          if (!from_in2 && !same_in) return bad("a phase without a hand-off must read what the previous phase staged", p);
          }
        } else if (leading) {
          return bad("a leading phase reads a staged input: FSVD_PF_NOWAIT must be set with FSVD_PF_LEAD", p);
        } else if (d.in_off != 0) {
          return bad("a staged input starts at offset 0", p);
        }
        if (stage2) {
          if (d.norm_w) return bad("two-vector staging applies the norm as a scalar: fold norm_w into the matrix", p);
          if (!d.in2.ptr || d.in2_len <= 0 || d.in2_len % 8 != 0 || d.in2_off % 8 != 0 || d.in2_off < n_in ||
              (int64_t)d.in2_off + d.in2_len > kMaxIn)
            return bad("second staged vector missing, misaligned, overlapping the first or past the staging buffer", p);
          if (((n_in / 2) + kT - 1) / kT + ((d.in2_len / 4) + kT - 1) / kT > 8) return bad("two-vector staging needs more than one round of loads", p);
        }
        const int64_t rows = ((int64_t)d.N + nwg - 1) / nwg;
        if (rows * d.nmat * (d.K / (q4 ? 256 : 128)) > kMaxChunks) return bad("too many rows per workgroup for the partial buffer", p);
        if (d.epilogue < 0 || d.epilogue > FSVD_EP_F32) return bad("unknown epilogue", p);
        if ((d.epilogue == FSVD_EP_SWIGLU) != (d.nmat == 2)) return bad("SwiGLU epilogue needs exactly two matrices", p);
        if (d.epilogue == FSVD_EP_RESID && !d.aux0.ptr) return bad("residual epilogue needs aux0", p);
        if (d.epilogue == FSVD_EP_RESID && rows > kT / 8) return bad("residual epilogue handles at most kT/8 rows per workgroup", p);
        if (split) {
          if (d.rows0 <= 0 || d.rows0 >= d.N) return bad("rows0 must cut the rows into two non-empty groups", p);
          if (d.epilogue != FSVD_EP_STORE && d.epilogue != FSVD_EP_RESID) return bad("the first row group stores or adds a residual", p);
        }
        if (f32rows) {
          if (d.nmat != 1) return bad("fp32 rows come from a single matrix", p);
          if (!d.out1.ptr) return bad("fp32 rows need out1", p);
          if ((d.aux2.ptr || split) && rows > kT / 8) return bad("a phase with two row groups or an addend handles at most kT/8 rows per workgroup", p);
        } else if (d.aux2.ptr || d.out1.ptr) {
          // aux2 / out1 overlay the attention pointers; a GEMV without fp32 rows must leave them empty
          return bad("aux2 / out1 without fp32 rows", p);
        }
        if ((rows + kU) * d.nmat * (d.K / (q4 ? 32 : 8)) * (int64_t)(d.K / (q4 ? 32 : 8)) >= (1ll << 32)) return bad("slab too large for the index arithmetic", p);
        if (d.epilogue == FSVD_EP_LOGITS && !d.plain_out) return bad("logits epilogue needs plain_out", p);
        if ((!nowait && !d.in.ptr) || (d.epilogue != FSVD_EP_F32 && !d.out0.ptr)) return bad("GEMV needs in and out0", p);
        for (int m = 0; m < d.nmat; ++m)
          if (reinterpret_cast<uintptr_t>(d.W[m]) & 15) return bad("weights must be 16-byte aligned", p);
        out0_written = d.epilogue != FSVD_EP_F32;
        out1_written = f32rows;
        break;
      }
      case FSVD_PH_ATTN: {
        if (d.Dh != 128) return bad("attention phase needs head_dim 128", p);
        if (d.H <= 0 || d.Hk <= 0 || d.H % d.Hk != 0) return bad("bad head counts", p);
        if (d.nsplit <= 0 || d.H * d.nsplit != nwg) return bad("H * nsplit must equal the workgroup count", p);
        if (!d.in.ptr || !d.out0.ptr || !d.k_cache || !d.v_cache) return bad("attention needs in = [q|k|v], out0 and the caches", p);
        // the producer is the grouped head expansion (H > 0, same geometry) or a plain GEMV of that many rows (a dense
        // [q; k; v] projection); phases without a hand-off may sit between the two
        const Seen* s = find(d.in.ptr);
        const fsvd_phase* pr = s ? &ph[s->last_write] : nullptr;
        if (!pr || pr->type != FSVD_PH_GEMV || pr->epilogue != FSVD_EP_STORE || (pr->flags & FSVD_PF_SPLIT) || pr->out0.ptr != d.in.ptr ||
            pr->N != (d.H + 2 * d.Hk) * d.Dh || (pr->H != 0 && (pr->H != d.H || pr->Hk != d.Hk || pr->Dh != d.Dh)))
          return bad("attention must read the output of the GEMV that writes (H + 2*Hk) * Dh values of q, k, v", p);
        for (int q = s->last_write + 1; q < p; ++q)
          if (ph[q].type != FSVD_PH_GEMV || !(ph[q].flags & FSVD_PF_NOWAIT)) return bad("only phases without a hand-off may sit between the q, k, v projection and its attention phase", p);
        if ((d.cos == nullptr) != (d.sin == nullptr) || (d.cos && d.rope_len <= 0)) return bad("rope tables incomplete", p);
        if ((d.sc_s % 8) || (d.sc_h % 8) || (reinterpret_cast<uintptr_t>(d.k_cache) & 15) || (reinterpret_cast<uintptr_t>(d.v_cache) & 15))
          return bad("cache strides/pointers must be 16-byte aligned", p);
        if (d.S <= 0) return bad("cache length missing", p);
        if (kSlots * (d.Dh + 2) + kSlots + 1 > kMaxChunks) return bad("internal: slot buffer", p);
        break;
      }
      case FSVD_PH_MERGE:
        if (p == 0 || ph[p - 1].type != FSVD_PH_ATTN) return bad("merge must follow an attention phase", p);
        if (d.H != ph[p - 1].H || d.Dh != ph[p - 1].Dh || d.nsplit != ph[p - 1].nsplit || d.in.ptr != ph[p - 1].out0.ptr)
          return bad("merge geometry differs from its attention phase", p);
        if (!d.out0.ptr || (d.H * d.Dh) % nwg != 0 || d.Dh % ((d.H * d.Dh) / nwg) != 0)
          return bad("merge needs out0 and H*Dh split evenly over the workgroups inside heads", p);
        if (d.nsplit * ((d.H * d.Dh) / nwg + 2) > kMaxChunks) return bad("internal: merge buffer", p);
        break;
      case FSVD_PH_ARGMAX:
        if (p == 0 || ph[p - 1].type != FSVD_PH_GEMV || ph[p - 1].epilogue != FSVD_EP_LOGITS || d.in.ptr != ph[p - 1].out0.ptr)
          return bad("argmax must follow a logits GEMV and read its candidates", p);
        if (p != nph - 1) return bad("argmax must be the last phase", p);
        out0_written = false;
        break;
      default:
        return bad("unknown phase type", p);
    }
    // every read must find its producer's tag schedule
    auto check_read = [&](const fsvd_tagbuf& r) -> const Seen* {
      const Seen* s = find(r.ptr);
      return (s && s->tb.uses_per_step == r.uses_per_step && s->tb.use == r.use) ? s : nullptr;
    };
    const bool nowait = d.type == FSVD_PH_GEMV && (d.flags & FSVD_PF_NOWAIT);
    if (d.type != FSVD_PH_EMBED && !nowait) {
      const Seen* s = check_read(d.in);
      if (!s) return bad("the input was not written by an earlier phase of the step, or with another tag schedule", p);
      if (d.type == FSVD_PH_GEMV) {
        // a fully polled input that every workgroup helped to write tells the reader that all of them are through its
        // producer; the two outputs of a phase with two row groups say so only together
        if (s->full) closes[p] = s->last_write;
        if (d.flags & FSVD_PF_STAGE2) {
          const Seen* s2 = check_read(d.in2);
          if (!s2) return bad("the second staged vector was not written by an earlier phase, or with another tag schedule", p);
          if (s2->full) closes[p] = std::max(closes[p], s2->last_write);
          if (s->half && s2->half && s->last_write == s2->last_write) closes[p] = std::max(closes[p], s->last_write);
        }
      }
    }
    if (d.type == FSVD_PH_GEMV) {
      if (d.epilogue == FSVD_EP_RESID && !check_read(d.aux0)) return bad("residual tag schedule differs from the producer's", p);
      if (d.aux2.ptr && !check_read(d.aux2)) return bad("addend tag schedule differs from the producer's", p);
    }
    // write-after-read safety: between two writes of one buffer every workgroup must be known to have finished reading
    // the old contents, i.e. some phase q in (last reader, this phase] has staged an input that closes a phase at or
    // behind the last reader (a phase stages before it writes, so q may be this phase itself).
    const fsvd_tagbuf* outs[2] = {out0_written ? &d.out0 : nullptr, out1_written ? &d.out1 : nullptr};
    for (const fsvd_tagbuf* ob : outs) {
      if (!ob || !ob->ptr) continue;
      const void* o = ob->ptr;
      if (ob->uses_per_step <= 0 || ob->use < 0 || ob->use >= ob->uses_per_step) return bad("bad tag schedule", p);
      const bool split = d.type == FSVD_PH_GEMV && (d.flags & FSVD_PF_SPLIT);
      Seen* s = find(o);
      if (!s) { seen.push_back({o, p, *ob, !split, split}); continue; }
      const int prev = s->last_write;
      int last_read = prev;
      for (int q = prev + 1; q <= p; ++q)
        if (reads(ph[q], o)) last_read = q;
      if (last_read == p) return bad("a phase must not write a buffer that it reads", p);
      bool closed = false;
      for (int q = last_read + 1; q <= p && !closed; ++q) closed = closes[q] >= last_read;
      if (!closed) return bad("buffer is rewritten before a full hand-off separates it from its last reader", p);
      *s = {o, p, *ob, !split, split};
    }
  }
  return kOk;
}

// Which build of the kernel a list needs: 0 plain bf16, 1 with the int4 code (~5 % slower on a bf16 list), 2 with the
// code of the composed form; + 4 for a float16 list (plain or composed).  A build that meets a phase it was not compiled
// for raises the step's error flag.
int decode_step_build(const fsvd_phase* host, int nph) {
  if (!host) return 0;
  int build = 0, f16 = 0;
  for (int p = 0; p < nph; ++p) {
    if (host[p].type != FSVD_PH_GEMV) continue;
    if (is_q4_bits(host[p].wbits)) build = 1;
    if (host[p].wbits == FSVD_WBITS_FP16 || host[p].wbits == FSVD_WBITS_Q4_FP16) f16 = 4;
    if (build != 1 && (host[p].flags != 0 || host[p].epilogue == FSVD_EP_F32)) build = 2;
  }
  return build + f16;
}

int launch_decode_step(const fsvd_phase* dev, int nph, fsvd_step_state* st, unsigned long long* trace, int trace_stride, int build,
                       hipStream_t stream) {
  const int nwg = decode_step_workgroups();
  if (nwg <= 0) return kErrLaunch;   // the reason is in the last-error text
  unsigned long long* tp = trace ? trace : nullptr;
  const int ts = trace ? trace_stride : 1;
#define FSVD_LAUNCH(T, Q, C, D) hipLaunchKernelGGL((decode_step_kernel<T, Q, C, D>), dim3(nwg), dim3(kT), kSmemBytes, stream, dev, nph, st, tp, ts)
  if (trace) {
    if (build == 1) FSVD_LAUNCH(true, true, false, 0);
    else if (build == 2) FSVD_LAUNCH(true, false, true, 0);
    else if (build == 4) FSVD_LAUNCH(true, false, false, 1);
    else if (build == 5) FSVD_LAUNCH(true, true, false, 1);
    else if (build == 6) FSVD_LAUNCH(true, false, true, 1);
    else FSVD_LAUNCH(true, false, false, 0);
  } else {
    if (build == 1) FSVD_LAUNCH(false, true, false, 0);
    else if (build == 2) FSVD_LAUNCH(false, false, true, 0);
    else if (build == 4) FSVD_LAUNCH(false, false, false, 1);
    else if (build == 5) FSVD_LAUNCH(false, true, false, 1);
    else if (build == 6) FSVD_LAUNCH(false, false, true, 1);
    else FSVD_LAUNCH(false, false, false, 0);
  }
#undef FSVD_LAUNCH
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("fsvd_decode_step: launch failed: %s", hipGetErrorString(e)); return kErrLaunch; }
  return kOk;
}

}  // namespace fsvd
