// Persistent batch-1 decode step: one workgroup per compute unit walks a list of phases.
//
// Hand-off between workgroups is by "tagged" vectors: a producer stores (tag << 16 | bf16) words with
// write-through agent-scope stores, a consumer polls the words it needs with agent-scope loads until
// every tag matches the tag expected for this use of the buffer.  Tags advance with every use, so stale
// contents never match, and there is no barrier object, counter or L2 write-back on the path.  Before a
// workgroup starts polling for the input of a phase it has already requested the first kU 16-byte
// pieces per lane of that phase's weights, so the HBM stream keeps running while the activations travel.
//
// Weight walk: a workgroup owns a "slab" of whole rows; the slab is cut into 16-byte pieces that are
// dealt to the 512 lanes in address order (fully coalesced); 16 consecutive lanes form a chunk (128
// elements of one row, K % 128 == 0) whose partial dot product is folded with DPP and parked in LDS;
// row sums add the chunks in order, so results do not depend on timing.
#include <cstddef>
#include <vector>

#include "../../include/flashsvd_hip.h"
#include "common.hpp"
#include "kernels.hpp"

namespace fsvd {

constexpr int kT = 512;                 // threads per workgroup
constexpr int kU = 10;                  // 16-byte weight pieces in flight per lane (rolling register window)
constexpr int kUA = kU / 2;             // attention: keys (and values) in flight per 16-lane slot
constexpr int kPoll = 12;               // 64-bit polls per lane per staging round
constexpr int kMaxIn = 16384;           // staged input elements (bf16) per phase
constexpr int kMaxChunks = 8192;        // chunk partials per workgroup per phase
constexpr int kSpinLimit = 1 << 20;     // polls before a workgroup gives up
constexpr int kSlots = kT / 16;         // 16-lane groups = keys in flight per load in the attention phase
constexpr size_t kSmemBytes = (size_t)kMaxIn * 2 + (size_t)kMaxChunks * 4 + 256;

__device__ __forceinline__ uint32_t tag16(int epoch, const fsvd_tagbuf& b) {
  return ((uint32_t)epoch * (uint32_t)b.uses_per_step + (uint32_t)b.use + 1u) & 0xffffu;
}
__device__ __forceinline__ uint32_t tag32(int epoch, const fsvd_tagbuf& b) {
  return (uint32_t)epoch * (uint32_t)b.uses_per_step + (uint32_t)b.use + 1u;
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
__device__ __forceinline__ u32x4_t ld_stream(const uint16_t* p) {
  return __builtin_nontemporal_load((gptr16_t)(uintptr_t)p);
}
__device__ __forceinline__ u32x4_t ld_global16(const uint16_t* p) { return *(gptr16_t)(uintptr_t)p; }

// poll one 64-bit word holding two tagged bf16 values; returns false on time-out / foreign error
__device__ __forceinline__ bool poll_pair(const void* buf, int idx64, uint32_t tag, const fsvd_step_state* st, int limit,
                                          uint32_t& lo, uint32_t& hi) {
  int spins = 0;
  for (;;) {
    const uint64_t v = ld_coh64(buf, idx64);
    lo = (uint32_t)v; hi = (uint32_t)(v >> 32);
    if ((lo >> 16) == tag && (hi >> 16) == tag) return true;
    if (++spins > limit) return false;
    if ((spins & 1023) == 0 && ld_err(st) != 0) return false;
  }
}
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
// weight slab of one workgroup for a GEMV / QKV phase
// ---------------------------------------------------------------------------------------------
// items are dealt share_q per workgroup plus one more for the first share_r workgroups
__device__ __forceinline__ int share_begin(const fsvd_phase& d, int w) { return w * d.share_q + min(w, d.share_r); }
__device__ __forceinline__ int share_count(const fsvd_phase& d, int w) { return d.share_q + (w < d.share_r ? 1 : 0); }

// A phase descriptor travels in one VGPR per lane (lane k holds 32-bit word k), loaded with a single
// coalesced read two phases ahead of its use; fields come out with readlane, i.e. without a dependent
// chain of scalar loads on the critical path.
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
__device__ __forceinline__ void* desc_ptr(uint32_t dv, int word) {
  return reinterpret_cast<void*>(((uint64_t)desc_u32(dv, word + 1) << 32) | desc_u32(dv, word));
}
__device__ __forceinline__ void desc_tagbuf(uint32_t dv, int word, fsvd_tagbuf& t) {
  t.ptr = desc_ptr(dv, word);
  t.uses_per_step = (int)desc_u32(dv, word + 2);
  t.use = (int)desc_u32(dv, word + 3);
}
__device__ __forceinline__ void desc_unpack(uint32_t dv, fsvd_phase& d) {
  d.type = (int)desc_u32(dv, FSVD_DW(type));
  d.epilogue = (int)desc_u32(dv, FSVD_DW(epilogue));
  d.N = (int)desc_u32(dv, FSVD_DW(N));
  d.K = (int)desc_u32(dv, FSVD_DW(K));
  d.nmat = (int)desc_u32(dv, FSVD_DW(nmat));
  d.mode = (int)desc_u32(dv, FSVD_DW(mode));
  d.H = (int)desc_u32(dv, FSVD_DW(H));
  d.Hk = (int)desc_u32(dv, FSVD_DW(Hk));
  d.Dh = (int)desc_u32(dv, FSVD_DW(Dh));
  d.nsplit = (int)desc_u32(dv, FSVD_DW(nsplit));
  d.rope_len = (int)desc_u32(dv, FSVD_DW(rope_len));
  d.S = (int)desc_u32(dv, FSVD_DW(S));
  d.fparam = __uint_as_float(desc_u32(dv, FSVD_DW(fparam)));
  d.W[0] = desc_ptr(dv, FSVD_DW(W));
  d.W[1] = desc_ptr(dv, FSVD_DW(W) + 2);
  d.W[2] = desc_ptr(dv, FSVD_DW(W) + 4);
  d.norm_w = desc_ptr(dv, FSVD_DW(norm_w));
  d.cos = desc_ptr(dv, FSVD_DW(cos));
  d.sin = desc_ptr(dv, FSVD_DW(sin));
  d.k_cache = desc_ptr(dv, FSVD_DW(k_cache));
  d.v_cache = desc_ptr(dv, FSVD_DW(v_cache));
  d.sc_s = (int64_t)reinterpret_cast<uintptr_t>(desc_ptr(dv, FSVD_DW(sc_s)));
  d.sc_h = (int64_t)reinterpret_cast<uintptr_t>(desc_ptr(dv, FSVD_DW(sc_h)));
  d.plain_out = desc_ptr(dv, FSVD_DW(plain_out));
  desc_tagbuf(dv, FSVD_DW(in), d.in);
  desc_tagbuf(dv, FSVD_DW(aux0), d.aux0);
  desc_tagbuf(dv, FSVD_DW(aux1), d.aux1);
  desc_tagbuf(dv, FSVD_DW(out0), d.out0);
  desc_tagbuf(dv, FSVD_DW(out1), d.out1);
  desc_tagbuf(dv, FSVD_DW(out2), d.out2);
  d.share_q = (int)desc_u32(dv, FSVD_DW(share_q));
  d.share_r = (int)desc_u32(dv, FSVD_DW(share_r));
  d.m_kp = desc_u32(dv, FSVD_DW(m_kp));
  d.m_pps = desc_u32(dv, FSVD_DW(m_pps));
}

struct Slab {
  int kind;                 // 0 contiguous rows of nmat matrices, 1 q/k/v row-pair units
  int nseg, srows, kp, pps, total, K;
  uint32_t m_kp, m_pps;     // reciprocals: n / kp = umulhi(n, m_kp), valid for n * kp < 2^32
  const uint16_t* b0; const uint16_t* b1;
  const uint16_t* Wq; const uint16_t* Wk; const uint16_t* Wv;
  int u0, gshift, nq, nk, Dh;
  int r0;                   // first output row (gemv)
};

__device__ __forceinline__ void qkv_unit(const Slab& s, int unit, int& m, int& head, int& g) {
  if (unit < s.nq) m = 0;
  else if (unit < s.nq + s.nk) { m = 1; unit -= s.nq; }
  else { m = 2; unit -= s.nq + s.nk; }
  head = unit >> s.gshift;
  g = unit - (head << s.gshift);
}
__device__ __forceinline__ const uint16_t* seg_ptr(const Slab& s, int seg) {
  if (s.kind == 0) return seg == 0 ? s.b0 : s.b1;
  int m, head, g;
  qkv_unit(s, s.u0 + (seg >> 1), m, head, g);
  const uint16_t* W = m == 0 ? s.Wq : (m == 1 ? s.Wk : s.Wv);
  return W + (int64_t)(head * s.Dh + g * 8 + (seg & 1) * (s.Dh >> 1)) * s.K;
}
__device__ __forceinline__ int seg_xoff(const Slab& s, int seg) {
  if (s.kind == 0) return seg * s.K;
  const int unit = s.u0 + (seg >> 1);
  return (unit < s.nq ? 0 : (unit < s.nq + s.nk ? 1 : 2)) * s.K;
}

__device__ __forceinline__ void slab_setup(const fsvd_phase& d, int w, int nwg, Slab& s) {
  s.K = d.K;
  s.kp = d.K >> 3;
  if (d.type == FSVD_PH_GEMV) {
    s.kind = 0;
    const int r0 = share_begin(d, w);
    s.r0 = r0;
    s.srows = share_count(d, w);
    s.nseg = d.nmat;
    s.b0 = static_cast<const uint16_t*>(d.W[0]) + (int64_t)r0 * d.K;
    s.b1 = d.nmat > 1 ? static_cast<const uint16_t*>(d.W[1]) + (int64_t)r0 * d.K : s.b0;
  } else {
    s.kind = 1;
    s.gshift = d.Dh == 128 ? 3 : 2;   // 8-row groups per half head: Dh / 16
    s.nq = d.H << s.gshift;
    s.nk = d.Hk << s.gshift;
    s.Dh = d.Dh;
    // a workgroup without a row group still requests (and drops) piece 0 of its slab: keep that inside
    // the matrices by pointing it at the last group
    s.u0 = min(share_begin(d, w), s.nq + 2 * s.nk - 1);
    s.nseg = 2 * share_count(d, w);
    s.srows = 8;
    s.Wq = static_cast<const uint16_t*>(d.W[0]);
    s.Wk = static_cast<const uint16_t*>(d.W[1]);
    s.Wv = static_cast<const uint16_t*>(d.W[2]);
    s.r0 = 0;
  }
  s.pps = s.srows * s.kp;
  s.total = s.nseg * s.pps;
  s.m_kp = d.m_kp;
  s.m_pps = d.m_pps;
}

// segment of piece i: contiguous slabs have at most two segments, q/k/v slabs short ones (8 rows)
__device__ __forceinline__ int seg_of(const Slab& s, int i) {
  return s.kind == 0 ? (i >= s.pps ? 1 : 0) : (int)__umulhi((uint32_t)i, s.m_pps);
}

// piece i of the slab (16 bytes): segment, offset inside the segment, position inside its row
__device__ __forceinline__ void slab_issue(const Slab& s, int i0, u32x4_t (&R)[kU]) {
#pragma unroll
  for (int u = 0; u < kU; ++u) {
    int i = i0 + u * kT + (int)threadIdx.x;
    i = i < s.total ? i : 0;
    const int seg = seg_of(s, i);
    const int rem = i - seg * s.pps;
    R[u] = ld_stream(seg_ptr(s, seg) + (int64_t)rem * 8);
  }
}
// consume the window for batch i0 and refill every slot with the same lane's piece of the next batch
// (RELOAD); pieces past the end of the slab clamp to piece 0, whose result is dropped
template <bool RELOAD>
__device__ __forceinline__ void slab_consume(const Slab& s, int i0, u32x4_t (&R)[kU], const uint16_t* xs, float* cp) {
#pragma unroll
  for (int u = 0; u < kU; ++u) {
    if (!RELOAD && i0 + u * kT >= s.total) break;   // the rest of the window lies past the slab (uniform)
    const int ir = i0 + u * kT + (int)threadIdx.x;
    const bool valid = ir < s.total;
    const int i = valid ? ir : 0;
    const int seg = seg_of(s, i);
    const int kofs = i - (int)__umulhi((uint32_t)i, s.m_kp) * s.kp;
    const u32x4_t xv = *reinterpret_cast<const u32x4_t*>(xs + seg_xoff(s, seg) + kofs * 8);
    float d = dot8_bf16(R[u], xv, 0.f);
    if (RELOAD) {
      int in = ir + kT * kU;
      in = in < s.total ? in : 0;
      const int segn = seg_of(s, in);
      R[u] = ld_stream(seg_ptr(s, segn) + (int64_t)(in - segn * s.pps) * 8);
    }
    d = row16_sum(d);
    if (valid && (threadIdx.x & 15) == 0) cp[i >> 4] = d;
  }
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

// ---------------------------------------------------------------------------------------------
// attention phase helpers: this workgroup = (head h, key split s) over the keys already cached
// ---------------------------------------------------------------------------------------------
struct AttnWork {
  int h, hk, s, k0, k1, newtok;
  const uint16_t* kbase; const uint16_t* vbase;
  int64_t sc_s;
};
__device__ __forceinline__ void attn_setup(const fsvd_phase& d, int w, int pos, AttnWork& a) {
  a.h = w / d.nsplit;
  a.s = w - a.h * d.nsplit;
  a.hk = a.h / (d.H / d.Hk);
  const int n_old = min(max(pos, 0), d.S);
  int per = (n_old + d.nsplit - 1) / d.nsplit;
  per = (per + kSlots - 1) / kSlots * kSlots;
  a.k0 = min(a.s * per, n_old);
  a.k1 = min(n_old, a.k0 + per);
  a.newtok = (a.s == d.nsplit - 1);
  const int part = threadIdx.x & 15;
  a.kbase = static_cast<const uint16_t*>(d.k_cache) + (int64_t)a.hk * d.sc_h + part * 8;
  a.vbase = static_cast<const uint16_t*>(d.v_cache) + (int64_t)a.hk * d.sc_h + part * 8;
  a.sc_s = d.sc_s;
}
__device__ __forceinline__ void attn_issue(const AttnWork& a, int c0, u32x4_t (&R)[kU]) {
  const int slot = threadIdx.x >> 4;
#pragma unroll
  for (int u = 0; u < kUA; ++u) {
    const int key = max(0, min(c0 + u * kSlots + slot, a.k1 - 1));
    R[u] = ld_global16(a.kbase + (int64_t)key * a.sc_s);
  }
#pragma unroll
  for (int u = 0; u < kUA; ++u) {
    const int key = max(0, min(c0 + u * kSlots + slot, a.k1 - 1));
    R[kUA + u] = ld_global16(a.vbase + (int64_t)key * a.sc_s);
  }
}
__device__ __forceinline__ void softmax_step(float sc, const u32x4_t& v, float& m, float& l, float (&acc)[8]) {
  const float m_new = fmaxf(m, sc);
  const float alpha = (m == -INFINITY) ? 0.f : __expf(m - m_new);
  const float p = __expf(sc - m_new);
  acc[0] = acc[0] * alpha + p * bf16_lo(v.x); acc[1] = acc[1] * alpha + p * bf16_hi(v.x);
  acc[2] = acc[2] * alpha + p * bf16_lo(v.y); acc[3] = acc[3] * alpha + p * bf16_hi(v.y);
  acc[4] = acc[4] * alpha + p * bf16_lo(v.z); acc[5] = acc[5] * alpha + p * bf16_hi(v.z);
  acc[6] = acc[6] * alpha + p * bf16_lo(v.w); acc[7] = acc[7] * alpha + p * bf16_hi(v.w);
  l = l * alpha + p;
  m = m_new;
}

// ---------------------------------------------------------------------------------------------
// request the first weights / keys of phase d (called before the workgroup polls for its input)
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ void prefetch_phase(const fsvd_phase& d, int w, int nwg, int pos, u32x4_t (&R)[kU]) {
  if (d.type == FSVD_PH_GEMV || d.type == FSVD_PH_QKV) {
    Slab slab;
    slab_setup(d, w, nwg, slab);
    slab_issue(slab, 0, R);
  } else if (d.type == FSVD_PH_ATTN) {
    AttnWork aw;
    attn_setup(d, w, pos, aw);
    attn_issue(aw, aw.k0, R);
  }
}

__device__ __forceinline__ void raise_error(fsvd_step_state* st, int p, int w) {
  if (threadIdx.x == 0) {
    __hip_atomic_store(&st->err, p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    st->err_wg = w;
  }
}

// poll the tagged input of a GEMV / QKV phase into LDS as packed bf16, RMS-normalised when asked
__device__ __forceinline__ bool stage_input(const fsvd_phase& d, uint32_t tin, const fsvd_step_state* st, int limit,
                                            uint16_t* xs, float* red) {
  const int tid = threadIdx.x;
  const int in_len = (d.type == FSVD_PH_QKV ? 3 : d.nmat) * d.K;
  const int nw64 = in_len >> 1;
  const bool norm = d.norm_w != nullptr;
  bool fail = false;
  float ss = 0.f;
  for (int base = 0; base < nw64; base += kT * kPoll) {
    uint32_t nwt[kPoll];
    if (norm) {
#pragma unroll
      for (int j = 0; j < kPoll; ++j) {
        const int q = base + j * kT + tid;
        nwt[j] = q < nw64 ? static_cast<const uint32_t*>(d.norm_w)[q] : 0u;
      }
    }
    uint64_t v[kPoll];
#pragma unroll
    for (int j = 0; j < kPoll; ++j) {
      const int q = base + j * kT + tid;
      v[j] = q < nw64 ? ld_coh64(d.in.ptr, q) : 0ull;
    }
#pragma unroll
    for (int j = 0; j < kPoll; ++j) {
      const int q = base + j * kT + tid;
      if (q < nw64) {
        uint32_t lo = (uint32_t)v[j], hi = (uint32_t)(v[j] >> 32);
        if ((lo >> 16) != tin || (hi >> 16) != tin) {
          if (!poll_pair(d.in.ptr, q, tin, st, limit, lo, hi)) fail = true;
        }
        lo &= 0xffffu;
        hi &= 0xffffu;
        if (norm) {
          const float a = bf16_bits_to_f32(lo), b = bf16_bits_to_f32(hi);
          ss += a * a + b * b;
          v[j] = ((uint64_t)hi << 32) | lo;   // raw values; scaled once the sum is known
        } else {
          reinterpret_cast<uint32_t*>(xs)[q] = lo | (hi << 16);
        }
      }
    }
    if (norm) {
      // normalised inputs fit one staging round (checked on the host)
      ss = wave_sum(ss);
      if ((tid & 63) == 0) red[tid >> 6] = ss;
      __syncthreads();
      float tot = 0.f;
#pragma unroll
      for (int i = 0; i < kT / 64; ++i) tot += red[i];
      const float rs = rsqrtf(tot / (float)in_len + d.fparam);
#pragma unroll
      for (int j = 0; j < kPoll; ++j) {
        const int q = base + j * kT + tid;
        if (q < nw64) {
          const float a = bf16_bits_to_f32((uint32_t)v[j]), b = bf16_bits_to_f32((uint32_t)(v[j] >> 32));
          reinterpret_cast<uint32_t*>(xs)[q] =
              pack_bf16x2(bf16_lo(nwt[j]) * round_bf16(a * rs), bf16_hi(nwt[j]) * round_bf16(b * rs));
        }
      }
    }
  }
  return !fail;
}

// TRACE: workgroups 0, stride, 2*stride, ... record wall-clock ticks (100 MHz) per phase:
// [0] phase entered, [1] input staged, [2] weights consumed, [3] epilogue done
template <bool TRACE>
__global__ __launch_bounds__(kT) void decode_step_kernel(const fsvd_phase* __restrict__ phases, int nph, fsvd_step_state* st,
                                                         unsigned long long* trace, int trace_stride) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  uint16_t* xs = reinterpret_cast<uint16_t*>(smem_raw);
  float* cp = reinterpret_cast<float*>(smem_raw + (size_t)kMaxIn * 2);
  float* red = cp + kMaxChunks;            // 32 floats
  int* ired = reinterpret_cast<int*>(red + 32);

  const int tid = threadIdx.x, w = blockIdx.x, nwg = gridDim.x;
  if (st->err != 0) return;
  const int epoch = st->epoch, pos = st->pos;
  const long long token = st->token;
  const int limit = st->spin_limit > 0 ? st->spin_limit : kSpinLimit;

  u32x4_t R[kU];
  uint32_t dvA = desc_fetch(phases, 0, nph), dvB = dvA;   // descriptors of phase p and p+1

  // Iteration p: finish streaming phase p (its first weights were requested one iteration earlier),
  // request the first weights of phase p+1, then run the epilogue of phase p while they travel.
  for (int p = -1; p < nph; ++p) {
    const uint32_t dvC = desc_fetch(phases, p + 2, nph);   // needed one iteration from now
    fsvd_phase d;
    desc_unpack(dvA, d);
    const int type = p < 0 ? -1 : d.type;
    unsigned long long* tr = nullptr;
    if (TRACE && p >= 0 && tid == 0 && (w % trace_stride) == 0) {
      tr = trace + ((size_t)(w / trace_stride) * nph + p) * 4;
      tr[0] = wall_clock64();
    }
    Slab slab;
    AttnWork aw;
    uint32_t resid = 0;
    float m_run = -INFINITY, l_run = 0.f;

    // ------------------------------------------------------------------ stage + stream
    if (type == FSVD_PH_GEMV || type == FSVD_PH_QKV) {
      slab_setup(d, w, nwg, slab);
      if (d.epilogue == FSVD_EP_RESID && (tid >> 3) < slab.srows) resid = ld_coh32(d.aux0.ptr, slab.r0 + (tid >> 3));
      const bool ok = stage_input(d, tag16(epoch, d.in), st, limit, xs, red);
      if (__syncthreads_or(ok ? 0 : 1)) { raise_error(st, p, w); return; }
      if (TRACE && tr) tr[1] = wall_clock64();
      const int nbatch = max(1, (slab.total + kT * kU - 1) / (kT * kU));
      for (int b = 0; b + 1 < nbatch; ++b) slab_consume<true>(slab, b * kT * kU, R, xs, cp);
      slab_consume<false>(slab, (nbatch - 1) * kT * kU, R, xs, cp);
      __syncthreads();
    } else if (type == FSVD_PH_ATTN) {
      // q of this head (and the new k, v for the split that owns the current token)
      attn_setup(d, w, pos, aw);
      const int Dh = d.Dh;   // 128: one key row = 16 lanes x 16 bytes
      const int w64 = Dh >> 1;
      bool fail = false;
      if (tid < 3 * w64) {
        const int which = tid / w64, q = tid - which * w64;
        if (which == 0 || aw.newtok) {
          const uint32_t tq = tag16(epoch, d.in), tk = tag16(epoch, d.aux0), tv = tag16(epoch, d.aux1);
          const void* buf = which == 0 ? d.in.ptr : (which == 1 ? d.aux0.ptr : d.aux1.ptr);
          const uint32_t tg = which == 0 ? tq : (which == 1 ? tk : tv);
          const int head = which == 0 ? aw.h : aw.hk;
          uint32_t lo, hi;
          if (!poll_pair(buf, head * w64 + q, tg, st, limit, lo, hi)) fail = true;
          reinterpret_cast<uint32_t*>(xs)[which * w64 + q] = (lo & 0xffffu) | (hi << 16);
        }
      }
      if (__syncthreads_or(fail ? 1 : 0)) { raise_error(st, p, w); return; }
      if (TRACE && tr) tr[1] = wall_clock64();
      const int part = tid & 15, slot = tid >> 4;
      const u32x4_t qv = *reinterpret_cast<const u32x4_t*>(xs + part * 8);
      float acc[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = 0.f;
      for (int c0 = aw.k0; c0 < aw.k1; c0 += kSlots * kUA) {
        if (c0 != aw.k0) attn_issue(aw, c0, R);
#pragma unroll
        for (int u = 0; u < kUA; ++u) {
          const float sc = row16_sum(dot8_bf16(R[u], qv, 0.f)) * d.fparam;
          if (c0 + u * kSlots + slot < aw.k1) softmax_step(sc, R[kUA + u], m_run, l_run, acc);
        }
      }
      if (aw.newtok && slot == 0) {
        const u32x4_t kn = *reinterpret_cast<const u32x4_t*>(xs + Dh + part * 8);
        const u32x4_t vn = *reinterpret_cast<const u32x4_t*>(xs + 2 * Dh + part * 8);
        const float sc = row16_sum(dot8_bf16(kn, qv, 0.f)) * d.fparam;
        softmax_step(sc, vn, m_run, l_run, acc);
      }
      // park the key slots: cp[slot][Dh + 2]
      float* sl = cp + slot * (Dh + 2);
#pragma unroll
      for (int i = 0; i < 8; ++i) sl[part * 8 + i] = acc[i];
      if (part == 0) { sl[Dh] = m_run; sl[Dh + 1] = l_run; }
      __syncthreads();
    }

    if (TRACE && tr) tr[2] = wall_clock64();
    // ------------------------------------------------------------------ first weights of the next phase
    // Phases whose epilogue polls (merge, argmax) or is trivial request the next weights first; GEMV / QKV
    // phases publish their outputs first (waves without output rows fall straight through to the request).
    const bool publish_first = (type == FSVD_PH_GEMV || type == FSVD_PH_QKV);
    if (!publish_first && p + 1 < nph) {
      fsvd_phase dn;
      desc_unpack(dvB, dn);
      prefetch_phase(dn, w, nwg, pos, R);
    }

    // ------------------------------------------------------------------ epilogue
    if (type == FSVD_PH_EMBED) {
      const int n0 = share_begin(d, w), n1 = n0 + share_count(d, w);
      const uint16_t* row = static_cast<const uint16_t*>(d.W[0]) + token * (int64_t)d.N;
      const uint32_t tg = tag16(epoch, d.out0);
      for (int n = n0 + tid; n < n1; n += kT) st_tag16(d.out0.ptr, n, tg, row[n]);
    } else if (type == FSVD_PH_GEMV) {
      const int cpr = slab.kp >> 4;
      const uint32_t tout = tag16(epoch, d.out0);
      const int grp = tid >> 3, lead = (tid & 7) == 0;
      const int npass = (slab.srows + kT / 8 - 1) / (kT / 8);
      if (d.epilogue == FSVD_EP_LOGITS) {
        float best = -INFINITY;
        int best_i = 0x7fffffff;
        for (int ps = 0; ps < npass; ++ps) {
          const int t = min(ps * (kT / 8) + grp, slab.srows - 1);
          const float v = round_bf16(row_sum8(cp, t, cpr));
          if (lead && ps * (kT / 8) + grp < slab.srows) {
            static_cast<uint16_t*>(d.plain_out)[slab.r0 + t] = (uint16_t)f32_to_bf16_bits(v);
            if (v > best) { best = v; best_i = slab.r0 + t; }
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
          const uint64_t word = ((uint64_t)((tout << 16) | f32_to_bf16_bits(best)) << 32) | (uint32_t)best_i;
          __hip_atomic_store(static_cast<uint64_t*>(d.out0.ptr) + w, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      } else if ((tid >> 6) * 8 < slab.srows) {   // waves whose lane groups own no row skip the epilogue
        for (int ps = 0; ps < npass; ++ps) {
          const int t = min(ps * (kT / 8) + grp, slab.srows - 1);
          const bool live = lead && ps * (kT / 8) + grp < slab.srows;
          const int n = slab.r0 + t;
          float v;
          if (d.epilogue == FSVD_EP_SWIGLU) {
            float gv = row_sum8(cp, t, cpr), uv = row_sum8(cp, slab.srows + t, cpr);
            if (d.mode == 0) {
              gv = round_bf16(gv);
              uv = round_bf16(uv);
              v = round_bf16(round_bf16(silu_f32(gv)) * uv);
            } else {
              v = round_bf16((gv * (1.0f / (1.0f + expf(-gv)))) * uv);
            }
          } else {
            v = round_bf16(row_sum8(cp, t, cpr));
            if (d.epilogue == FSVD_EP_RESID) v = round_bf16(bf16_bits_to_f32(resid & 0xffffu) + v);
          }
          if (live) st_tag16(d.out0.ptr, n, tout, f32_to_bf16_bits(v));
        }
      }
      // no barrier here: the next phase writes cp only after its staging barrier, which every wave reaches
      // after this epilogue; `red` is touched by the logits epilogue alone
      if (d.epilogue == FSVD_EP_LOGITS) __syncthreads();
    } else if (type == FSVD_PH_QKV) {
      // q/k/v row pairs: rotate-half RoPE in eager bf16 arithmetic, tagged q/k/v for the attention
      // phase and the cache append for later steps
      const int cpr = slab.kp >> 4;
      const int half = d.Dh >> 1;
      const int npair = (slab.nseg >> 1) * 8;
      const uint32_t tq = tag16(epoch, d.out0), tk = tag16(epoch, d.out1), tv = tag16(epoch, d.out2);
      for (int t0 = 0; t0 < npair && (tid >> 6) * 8 < npair; t0 += kT / 8) {
        const int t = min(t0 + (tid >> 3), npair - 1);
        const bool live = (tid & 7) == 0 && t0 + (tid >> 3) < npair;
        const int ul = t >> 3, r = t & 7;
        int m, head, g;
        qkv_unit(slab, slab.u0 + ul, m, head, g);
        const int dd = g * 8 + r;
        float x0 = round_bf16(row_sum8(cp, ul * 16 + r, cpr)), x1 = round_bf16(row_sum8(cp, ul * 16 + 8 + r, cpr));
        if (!live) continue;
        if (m != 2 && d.cos) {
          const int tp = min(max(pos, 0), d.rope_len - 1);
          const float c = bf16_bits_to_f32(static_cast<const uint16_t*>(d.cos)[(int64_t)tp * half + dd]);
          const float sn = bf16_bits_to_f32(static_cast<const uint16_t*>(d.sin)[(int64_t)tp * half + dd]);
          const float r0 = round_bf16(round_bf16(x0 * c) - round_bf16(x1 * sn));
          const float r1 = round_bf16(round_bf16(x1 * c) + round_bf16(x0 * sn));
          x0 = r0; x1 = r1;
        }
        const uint32_t o0 = f32_to_bf16_bits(x0), o1 = f32_to_bf16_bits(x1);
        const int e = head * d.Dh + dd;
        if (m == 0) {
          st_tag16(d.out0.ptr, e, tq, o0);
          st_tag16(d.out0.ptr, e + half, tq, o1);
        } else {
          st_tag16(m == 1 ? d.out1.ptr : d.out2.ptr, e, m == 1 ? tk : tv, o0);
          st_tag16(m == 1 ? d.out1.ptr : d.out2.ptr, e + half, m == 1 ? tk : tv, o1);
          if (pos >= 0 && pos < d.S) {
            uint16_t* cb = static_cast<uint16_t*>(m == 1 ? d.k_cache : d.v_cache) + (int64_t)pos * d.sc_s +
                           (int64_t)head * d.sc_h + dd;
            cb[0] = (uint16_t)o0;
            cb[half] = (uint16_t)o1;
          }
        }
      }
    } else if (type == FSVD_PH_ATTN) {
      // fold the key slots and publish this split's (acc, m, l)
      const int Dh = d.Dh;
      float* wts = cp + kSlots * (Dh + 2);
      float M = -INFINITY;
      for (int j = 0; j < kSlots; ++j) M = fmaxf(M, cp[j * (Dh + 2) + Dh]);
      if (tid < kSlots) {
        const float mj = cp[tid * (Dh + 2) + Dh];
        wts[tid] = (mj == -INFINITY) ? 0.f : __expf(mj - M);
      }
      __syncthreads();
      if (tid < Dh + 2) {
        float o = M;
        if (tid != Dh) {
          const int col = tid < Dh ? tid : Dh + 1;
          o = 0.f;
#pragma unroll 8
          for (int j = 0; j < kSlots; ++j) o += wts[j] * cp[j * (Dh + 2) + col];
        }
        st_tag64(d.out0.ptr, (aw.h * d.nsplit + aw.s) * (Dh + 2) + tid, tag32(epoch, d.out0), __float_as_uint(o));
      }
      __syncthreads();   // the merge phase reuses cp without a barrier of its own in front
    } else if (type == FSVD_PH_MERGE) {
      // merge the key splits: this workgroup owns `cnt` consecutive output elements of one head; one
      // lane polls one word (cnt accumulators + m + l for every split), so all polls are in flight at once
      const int cnt = d.share_q;                 // H * Dh / workgroups
      const int o0 = w * cnt;
      const int dsh = d.Dh == 128 ? 7 : 6;
      const int head = o0 >> dsh, dim0 = o0 - (head << dsh);
      const uint32_t tin = tag32(epoch, d.in), tout = tag16(epoch, d.out0);
      const int per = cnt + 2, items = d.nsplit * per;
      bool fail = false;
      for (int it = tid; it < items; it += kT) {
        const int sp = it / per, j = it - sp * per;
        const int col = j < cnt ? dim0 + j : d.Dh + (j - cnt);
        uint32_t payload;
        if (!poll_w64(d.in.ptr, (head * d.nsplit + sp) * (d.Dh + 2) + col, tin, st, limit, payload)) fail = true;
        cp[it] = __uint_as_float(payload);
      }
      if (__syncthreads_or(fail ? 1 : 0)) { raise_error(st, p, w); return; }
      if (tid < cnt) {
        float M = -INFINITY, num = 0.f, den = 0.f;
        for (int sp = 0; sp < d.nsplit; ++sp) M = fmaxf(M, cp[sp * per + cnt]);
        for (int sp = 0; sp < d.nsplit; ++sp) {
          const float mi = cp[sp * per + cnt];
          const float wi = (mi == -INFINITY) ? 0.f : __expf(mi - M);
          num += wi * cp[sp * per + tid];
          den += wi * cp[sp * per + cnt + 1];
        }
        st_tag16(d.out0.ptr, o0 + tid, tout, f32_to_bf16_bits(den > 0.f ? num / den : 0.f));
      }
    } else if (type == FSVD_PH_ARGMAX) {
      // greedy token, state advance
      if (w == 0) {
        const uint32_t tin = tag16(epoch, d.in);
        float best = -INFINITY;
        int best_i = 0x7fffffff;
        bool fail = false;
        for (int t = tid; t < nwg; t += kT) {
          int spins = 0;
          for (;;) {
            const uint64_t v = ld_coh64(d.in.ptr, t);
            if ((uint32_t)(v >> 48) == tin) {
              const float val = bf16_bits_to_f32((uint32_t)(v >> 32) & 0xffffu);
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
        if (__syncthreads_or(fail ? 1 : 0)) { raise_error(st, p, w); return; }
        if (tid == 0) {
          for (int i = 1; i < kT / 64; ++i)
            if (red[i] > best || (red[i] == best && ired[i] < best_i)) { best = red[i]; best_i = ired[i]; }
          if (d.plain_out) static_cast<long long*>(d.plain_out)[st->step] = best_i;
          st->token = best_i;
          st->pos = pos + 1;
          st->step = st->step + 1;
        }
      }
    }
    if (TRACE && tr) tr[3] = wall_clock64();
    if (publish_first && p + 1 < nph) {
      fsvd_phase dn;
      desc_unpack(dvB, dn);
      prefetch_phase(dn, w, nwg, pos, R);
    }
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

int decode_step_workgroups() {
  if (g_step_wgs > 0) return g_step_wgs;
  int dev = 0;
  hipDeviceProp_t prop;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 0;
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(decode_step_kernel<false>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)kSmemBytes) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(decode_step_kernel<true>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)kSmemBytes) != hipSuccess)
      return 0;
    attr_set = true;
  }
  g_step_wgs = prop.multiProcessorCount;
  return g_step_wgs;
}

int prepare_decode_step(fsvd_phase* ph, int nph, int nwg) {
  for (int p = 0; p < nph; ++p) {
    fsvd_phase& d = ph[p];
    int items = 0;
    if (d.type == FSVD_PH_EMBED || d.type == FSVD_PH_GEMV) items = d.N;
    else if (d.type == FSVD_PH_QKV) items = (d.H + 2 * d.Hk) * (d.Dh / 16);
    else if (d.type == FSVD_PH_MERGE) items = d.H * d.Dh;
    d.share_q = items / nwg;
    d.share_r = items % nwg;
    d.m_kp = d.m_pps = 0;
    if ((d.type == FSVD_PH_GEMV || d.type == FSVD_PH_QKV) && d.K >= 8) {
      d.m_kp = 0xffffffffu / (uint32_t)(d.K / 8) + 1u;
      d.m_pps = 0xffffffffu / (uint32_t)(d.K) + 1u;   // q/k/v segments are 8 rows: 8 * K / 8 pieces
    }
  }
  return kOk;
}

static int bad(const char* what, int p) {
  set_last_error("fsvd_decode_step: phase %d: %s", p, what);
  return kErrBadShape;
}

int validate_decode_step(const fsvd_phase* ph, int nph, int nwg) {
  if (nph < 2) return bad("a step needs at least two phases", 0);
  // last phase index that wrote each buffer and whether a "closing" GEMV consumed a fully-shared vector since
  struct Seen { const void* ptr; int last_write; fsvd_tagbuf tb; };
  std::vector<Seen> seen;
  std::vector<char> writes_all(nph, 0);
  for (int p = 0; p < nph; ++p) {
    const fsvd_phase& d = ph[p];
    {
      int items = 0;
      if (d.type == FSVD_PH_EMBED || d.type == FSVD_PH_GEMV) items = d.N;
      else if (d.type == FSVD_PH_QKV) items = (d.H + 2 * d.Hk) * (d.Dh / 16);
      else if (d.type == FSVD_PH_MERGE) items = d.H * d.Dh;
      if (d.share_q != items / nwg || d.share_r != items % nwg) return bad("derived fields missing: call fsvd_decode_step_prepare", p);
      if ((d.type == FSVD_PH_GEMV || d.type == FSVD_PH_QKV) && d.K >= 8 &&
          (d.m_kp != 0xffffffffu / (uint32_t)(d.K / 8) + 1u || d.m_pps != 0xffffffffu / (uint32_t)d.K + 1u))
        return bad("derived fields missing: call fsvd_decode_step_prepare", p);
    }
    switch (d.type) {
      case FSVD_PH_EMBED:
        if (!d.W[0] || !d.out0.ptr || d.N < nwg) return bad("embedding phase needs W[0], out0 and N >= workgroups", p);
        writes_all[p] = 1;
        break;
      case FSVD_PH_GEMV: {
        if (d.nmat < 1 || d.nmat > 2 || !d.W[0] || (d.nmat == 2 && !d.W[1])) return bad("GEMV needs 1 or 2 matrices", p);
        if (d.K <= 0 || d.K % 128 != 0) return bad("K must be a positive multiple of 128", p);
        if (d.N < nwg) return bad("fewer rows than workgroups", p);
        if (d.nmat * d.K > kMaxIn) return bad("input vector longer than the staging buffer", p);
        if (d.norm_w && d.nmat * d.K > kT * kPoll * 2) return bad("normalised input too long for one staging round", p);
        const int64_t rows = ((int64_t)d.N + nwg - 1) / nwg;
        if (rows * d.nmat * (d.K / 128) > kMaxChunks) return bad("too many rows per workgroup for the partial buffer", p);
        if ((d.epilogue == FSVD_EP_SWIGLU) != (d.nmat == 2)) return bad("SwiGLU epilogue needs exactly two matrices", p);
        if (d.epilogue == FSVD_EP_RESID && !d.aux0.ptr) return bad("residual epilogue needs aux0", p);
        if (d.epilogue == FSVD_EP_RESID && rows > kT / 8) return bad("residual epilogue handles at most 64 rows per workgroup", p);
        if (rows * d.nmat * (d.K / 8) * (int64_t)(d.K / 8) >= (1ll << 32)) return bad("slab too large for the index arithmetic", p);
        if (d.epilogue == FSVD_EP_LOGITS && !d.plain_out) return bad("logits epilogue needs plain_out", p);
        if (d.epilogue < 0 || d.epilogue > FSVD_EP_LOGITS) return bad("unknown epilogue", p);
        if (!d.in.ptr || !d.out0.ptr) return bad("GEMV needs in and out0", p);
        for (int m = 0; m < d.nmat; ++m)
          if (reinterpret_cast<uintptr_t>(d.W[m]) & 15) return bad("weights must be 16-byte aligned", p);
        writes_all[p] = 1;
        break;
      }
      case FSVD_PH_QKV: {
        if (d.Dh != 128 && d.Dh != 64) return bad("head_dim must be 64 or 128", p);
        if (d.H <= 0 || d.Hk <= 0 || d.H % d.Hk != 0) return bad("bad head counts", p);
        if (d.K <= 0 || d.K % 128 != 0) return bad("q/k/v ranks must be equal multiples of 128", p);
        if (3 * d.K > kMaxIn) return bad("input vector longer than the staging buffer", p);
        const int nu = (d.H + 2 * d.Hk) * (d.Dh / 16);
        const int64_t upw = ((int64_t)nu + nwg - 1) / nwg;
        if (upw * 16 * (d.K / 128) > kMaxChunks) return bad("too many rows per workgroup for the partial buffer", p);
        if (!d.W[0] || !d.W[1] || !d.W[2] || !d.in.ptr || !d.out0.ptr || !d.out1.ptr || !d.out2.ptr || !d.k_cache || !d.v_cache)
          return bad("QKV needs three matrices, in, out0..2 and the caches", p);
        if (d.cos && (!d.sin || d.rope_len <= 0)) return bad("rope tables incomplete", p);
        if (d.S <= 0) return bad("cache length missing", p);
        writes_all[p] = nu >= nwg;   // with fewer row groups than workgroups some workgroups only pass through
        break;
      }
      case FSVD_PH_ATTN:
        if (d.Dh != 128) return bad("attention phase needs head_dim 128", p);
        if (d.H <= 0 || d.Hk <= 0 || d.H % d.Hk != 0) return bad("bad head counts", p);
        if (d.nsplit <= 0 || d.H * d.nsplit != nwg) return bad("H * nsplit must equal the workgroup count", p);
        if (!d.in.ptr || !d.aux0.ptr || !d.aux1.ptr || !d.out0.ptr || !d.k_cache || !d.v_cache) return bad("attention needs q, new k/v, out0, caches", p);
        if ((d.sc_s % 8) || (d.sc_h % 8) || (reinterpret_cast<uintptr_t>(d.k_cache) & 15) || (reinterpret_cast<uintptr_t>(d.v_cache) & 15))
          return bad("cache strides/pointers must be 16-byte aligned", p);
        if (d.S <= 0) return bad("cache length missing", p);
        if (kSlots * (d.Dh + 2) + kSlots > kMaxChunks) return bad("internal: slot buffer", p);
        writes_all[p] = 1;
        break;
      case FSVD_PH_MERGE:
        if (p == 0 || ph[p - 1].type != FSVD_PH_ATTN) return bad("merge must follow an attention phase", p);
        if (d.H != ph[p - 1].H || d.Dh != ph[p - 1].Dh || d.nsplit != ph[p - 1].nsplit || d.in.ptr != ph[p - 1].out0.ptr)
          return bad("merge geometry differs from its attention phase", p);
        if (!d.out0.ptr || (d.H * d.Dh) % nwg != 0 || d.Dh % ((d.H * d.Dh) / nwg) != 0)
          return bad("merge needs out0 and H*Dh split evenly over the workgroups inside heads", p);
        if (d.nsplit * ((d.H * d.Dh) / nwg + 2) > kMaxChunks) return bad("internal: merge buffer", p);
        writes_all[p] = 1;
        break;
      case FSVD_PH_ARGMAX:
        if (p == 0 || ph[p - 1].type != FSVD_PH_GEMV || ph[p - 1].epilogue != FSVD_EP_LOGITS || d.in.ptr != ph[p - 1].out0.ptr)
          return bad("argmax must follow a logits GEMV and read its candidates", p);
        if (p != nph - 1) return bad("argmax must be the last phase", p);
        break;
      default:
        return bad("unknown phase type", p);
    }
    // every read must find its producer's tag schedule
    auto check_read = [&](const fsvd_tagbuf& r) -> bool {
      for (auto& s : seen)
        if (s.ptr == r.ptr) return s.tb.uses_per_step == r.uses_per_step && s.tb.use == r.use;
      return false;
    };
    if (d.type != FSVD_PH_EMBED) {
      if (p == 0 || d.in.ptr != ph[p - 1].out0.ptr) return bad("a phase must read the previous phase's out0", p);
      if (!check_read(d.in)) return bad("input tag schedule differs from the producer's", p);
      if (d.type == FSVD_PH_GEMV && d.epilogue == FSVD_EP_RESID && !check_read(d.aux0))
        return bad("residual tag schedule differs from the producer's", p);
      if (d.type == FSVD_PH_ATTN && (!check_read(d.aux0) || !check_read(d.aux1)))
        return bad("new k/v tag schedule differs from the producer's", p);
    } else if (p != 0) {
      return bad("the embedding phase must come first", p);
    }
    // write-after-read safety: between two writes of one buffer there must be a GEMV/QKV phase (which reads
    // its whole input) whose input every workgroup helped to write, and that phase must come after the
    // last reader of the old contents (readers are the next phase, or a residual / attention aux read).
    const fsvd_tagbuf* outs[3] = {&d.out0, d.type == FSVD_PH_QKV ? &d.out1 : nullptr, d.type == FSVD_PH_QKV ? &d.out2 : nullptr};
    for (const fsvd_tagbuf* ob : outs) {
      if (!ob || !ob->ptr) continue;
      void* o = ob->ptr;
      if (ob->uses_per_step <= 0 || ob->use < 0 || ob->use >= ob->uses_per_step) return bad("bad tag schedule", p);
      int prev = -1;
      for (auto& s : seen)
        if (s.ptr == o) { prev = s.last_write; s.last_write = p; s.tb = *ob; }
      if (prev < 0) { seen.push_back({o, p, *ob}); continue; }
      // last reader of the previous contents
      int last_read = prev + 1;
      for (int q = prev + 1; q < p; ++q)
        if (ph[q].in.ptr == o || ph[q].aux0.ptr == o || ph[q].aux1.ptr == o) last_read = q;
      bool closed = false;
      for (int q = last_read + 1; q <= p && !closed; ++q)
        if ((ph[q].type == FSVD_PH_GEMV || ph[q].type == FSVD_PH_QKV) && q > 0 && writes_all[q - 1] && q - 1 >= last_read) closed = true;
      if (!closed) return bad("buffer is rewritten before a full hand-off separates it from its last reader", p);
    }
  }
  return kOk;
}

int launch_decode_step(const fsvd_phase* dev, int nph, fsvd_step_state* st, unsigned long long* trace, int trace_stride,
                       hipStream_t stream) {
  const int nwg = decode_step_workgroups();
  if (nwg <= 0) { set_last_error("fsvd_decode_step: cannot query the device"); return kErrLaunch; }
  if (trace) hipLaunchKernelGGL(decode_step_kernel<true>, dim3(nwg), dim3(kT), kSmemBytes, stream, dev, nph, st, trace, trace_stride);
  else hipLaunchKernelGGL(decode_step_kernel<false>, dim3(nwg), dim3(kT), kSmemBytes, stream, dev, nph, st, nullptr, 1);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("fsvd_decode_step: launch failed: %s", hipGetErrorString(e)); return kErrLaunch; }
  return kOk;
}

}  // namespace fsvd
