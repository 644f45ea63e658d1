// Single-query attention over a dense KV cache [B,S,Hk,Dh] (K stored post-RoPE), split over
// the key axis so that B*H*nsplit workgroups cover the chip.  Each workgroup scores its key
// range in passes of 128 keys: every K and V row of a pass is requested up front (16-byte loads,
// 16 in flight per lane), scores come from V_DOT2 against the query chunk held in registers with
// a DPP fold over the lanes that share a key, the softmax is the online (running max / sum)
// form and p*V accumulates per lane.  The workgroup writes an un-normalised partial (acc, m, l)
// with write-through stores; the last workgroup to arrive for a (b,h) merges the partials in
// split order, so the result does not depend on arrival order.
#include "common.hpp"
#include "kernels.hpp"

namespace fsvd {

constexpr int kAttnThreads = 256;
constexpr int kMaxKeysPerSplit = 1 << 20;  // the key loop is streamed; only a sanity bound

__device__ __forceinline__ void decode_work_item(int B, int H, int nsplit, int& b, int& h, int& s) {
  // Consecutive workgroup ids go round-robin over the 8 XCDs; remap so that the splits of one
  // head (which meet again in the merge) run on the same XCD and share its L2.
  const int total = B * H * nsplit;
  int id = blockIdx.x;
  if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
  s = id % nsplit;
  h = (id / nsplit) % H;
  b = id / (nsplit * H);
}

// coherent (L2-bypassing) scalar accessors for the cross-workgroup partials: the producers write
// through to memory and the merging workgroup reads from memory, so no L2 write-back / invalidate
// fence is needed (those serialise per XCD and cost more than the whole kernel)
__device__ __forceinline__ void st_agent(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float ld_agent(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

template <int DT, int DH, int U>
__global__ __launch_bounds__(kAttnThreads) void attn_decode_kernel(AttnDecodeArgs a) {
  typedef E16<DT> E;
  constexpr int LPK = DH / 8;                 // lanes that share one key (8 bf16 each)
  constexpr int KPB = kAttnThreads / LPK;     // keys per block pass
  constexpr int CH = KPB * U;                 // keys in flight per workgroup
  __shared__ __align__(16) float accs[KPB * DH];
  __shared__ __align__(16) uint16_t qs[DH];
  __shared__ float red[2][4];
  __shared__ int last_flag;

  int b, h, s;
  decode_work_item(a.B, a.H, a.nsplit, b, h, s);
  const int tid = threadIdx.x;
  const int hk = h / (a.H / a.Hk);
  int n_keys = a.seqlens[b] + a.seqlen_add;
  n_keys = max(0, min(n_keys, a.S));
  int per = (n_keys + a.nsplit - 1) / a.nsplit;
  per = (per + KPB - 1) / KPB * KPB;
  const int k0 = min(s * per, n_keys);
  const int k1 = min(n_keys, k0 + per);

  // query chunk (optionally rotated at position seqlens[b], fp32 math, one rounding)
  const uint16_t* qp = a.q + (int64_t)b * a.sq_b + (int64_t)h * a.sq_h;
  if (tid < DH / 2) {
    float x0 = E::val(qp[tid]), x1 = E::val(qp[tid + DH / 2]);
    if (a.cos) {
      const int tp = min(max(a.seqlens[b], 0), a.rope_len - 1);
      const float c = E::val(a.cos[(int64_t)tp * (DH / 2) + tid]);
      const float sn = E::val(a.sin[(int64_t)tp * (DH / 2) + tid]);
      const float r0 = x0 * c - x1 * sn, r1 = x0 * sn + x1 * c;
      x0 = r0; x1 = r1;
    }
    qs[tid] = (uint16_t)E::bits(x0);
    qs[tid + DH / 2] = (uint16_t)E::bits(x1);
  }
  const int part = tid % LPK, slot = tid / LPK;
  const uint16_t* kbase = a.k_cache + (int64_t)b * a.sc_b + (int64_t)hk * a.sc_h + part * 8;
  const uint16_t* vbase = a.v_cache + (int64_t)b * a.sc_b + (int64_t)hk * a.sc_h + part * 8;

  float m_run = -INFINITY, l_thr = 0.f;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  int it = 0;
  for (int c0 = k0; c0 < k1; c0 += CH, ++it) {
    // all K and V rows of this pass are requested before anything is consumed
    u32x4_t kv[U], vv[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int key = min(c0 + u * KPB + slot, k1 - 1);
      kv[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(kbase + (int64_t)key * a.sc_s));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int key = min(c0 + u * KPB + slot, k1 - 1);
      vv[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(vbase + (int64_t)key * a.sc_s));
    }
    if (it == 0) __syncthreads();  // qs ready
    const u32x4_t qv = *reinterpret_cast<const u32x4_t*>(qs + part * 8);
    float sc[U];
    float lmax = -INFINITY;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float d = E::dot8(kv[u], qv, 0.f);
      d += dpp_f32<0xB1>(d);
      d += dpp_f32<0x4E>(d);
      d += dpp_f32<0x141>(d);
      if (LPK == 16) d += dpp_f32<0x140>(d);
      sc[u] = (c0 + u * KPB + slot < k1) ? d * a.scale : -INFINITY;
      lmax = fmaxf(lmax, sc[u]);
    }
    lmax = wave_max(lmax);
    const int rb = it & 1;
    if ((tid & 63) == 0) red[rb][tid >> 6] = lmax;
    __syncthreads();
    const float m_c = fmaxf(fmaxf(red[rb][0], red[rb][1]), fmaxf(red[rb][2], red[rb][3]));
    const float m_new = fmaxf(m_run, m_c);
    const float alpha = (m_run == -INFINITY) ? 0.f : __expf(m_run - m_new);
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] *= alpha;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float p = (sc[u] == -INFINITY) ? 0.f : __expf(sc[u] - m_new);
      psum += p;
      acc[0] += p * E::lo(vv[u].x); acc[1] += p * E::hi(vv[u].x);
      acc[2] += p * E::lo(vv[u].y); acc[3] += p * E::hi(vv[u].y);
      acc[4] += p * E::lo(vv[u].z); acc[5] += p * E::hi(vv[u].z);
      acc[6] += p * E::lo(vv[u].w); acc[7] += p * E::hi(vv[u].w);
    }
    l_thr = l_thr * alpha + (part == 0 ? psum : 0.f);
    m_run = m_new;
  }
  if (it == 0) __syncthreads();
  // fold the key slots and the per-thread sums
#pragma unroll
  for (int i = 0; i < 8; ++i) accs[slot * DH + part * 8 + i] = acc[i];
  float lw = wave_sum(l_thr);
  __syncthreads();  // red[] of the last pass consumed; accs written
  if ((tid & 63) == 0) red[0][tid >> 6] = lw;
  __syncthreads();
  const float l = (red[0][0] + red[0][1]) + (red[0][2] + red[0][3]);
  const float m = m_run;
  float o = 0.f;
  if (tid < DH) {
#pragma unroll 8
    for (int j = 0; j < KPB; ++j) o += accs[j * DH + tid];
  }

  uint16_t* outp = a.out + (int64_t)b * a.so_b + (int64_t)h * a.so_h;
  if (a.nsplit == 1) {
    if (tid < DH) outp[tid] = (uint16_t)E::bits(l > 0.f ? o / l : 0.f);
    return;
  }
  float* part_ws = a.ws_part + ((int64_t)(b * a.H + h) * a.nsplit) * (DH + 2);
  float* mine = part_ws + (int64_t)s * (DH + 2);
  if (tid < DH) st_agent(mine + tid, o);
  if (tid == 0) { st_agent(mine + DH, m); st_agent(mine + DH + 1, l); }
  wait_stores_acked();
  __syncthreads();
  if (tid == 0) {
    const int old = __hip_atomic_fetch_add(&a.ws_count[b * a.H + h], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last_flag = (old == a.nsplit - 1);
  }
  __syncthreads();
  if (!last_flag) return;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  if (tid < DH) {
    // the loads of eight splits are in flight at once (each comes from beyond this XCD's L2; one split per round trip
    // made this merge a third of the kernel at eight splits); the splits are added in order
    constexpr int SU = 8;
    float M = -INFINITY;
    for (int i0 = 0; i0 < a.nsplit; i0 += SU) {
      float mi[SU];
#pragma unroll
      for (int u = 0; u < SU; ++u) mi[u] = ld_agent(part_ws + (int64_t)min(i0 + u, a.nsplit - 1) * (DH + 2) + DH);
#pragma unroll
      for (int u = 0; u < SU; ++u) M = fmaxf(M, mi[u]);
    }
    float num = 0.f, den = 0.f;
    for (int i0 = 0; i0 < a.nsplit; i0 += SU) {
      float mi[SU], oi[SU], li[SU];
#pragma unroll
      for (int u = 0; u < SU; ++u) {
        const float* pw = part_ws + (int64_t)min(i0 + u, a.nsplit - 1) * (DH + 2);
        mi[u] = ld_agent(pw + DH);
        oi[u] = ld_agent(pw + tid);
        li[u] = ld_agent(pw + DH + 1);
      }
#pragma unroll
      for (int u = 0; u < SU; ++u) {
        const float w = (i0 + u >= a.nsplit || mi[u] == -INFINITY) ? 0.f : __expf(mi[u] - M);
        num += w * oi[u];
        den += w * li[u];
      }
    }
    outp[tid] = (uint16_t)E::bits(den > 0.f ? num / den : 0.f);
  }
  if (tid == 0) __hip_atomic_store(&a.ws_count[b * a.H + h], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Grouped-query caches: G query heads of one kv head per workgroup.  The K and V rows of a pass are requested once and
// scored against the G queries (with one workgroup per query head every head of a group re-reads its kv head's rows from
// L2); running maximum, sum and accumulators per query head; the heads' partials and merges go one after the other
// through the same LDS block and the same last-arriver protocol as above.  G divides H / Hk.
template <int DT, int DH, int U, int G>
__global__ __launch_bounds__(kAttnThreads) void attn_decode_gqa_kernel(AttnDecodeArgs a) {
  typedef E16<DT> E;
  constexpr int LPK = DH / 8, KPB = kAttnThreads / LPK, CH = KPB * U;
  static_assert(G * DH / 2 <= kAttnThreads, "one thread per rotation pair of every query of the group");
  __shared__ __align__(16) float accs[KPB * DH];
  __shared__ __align__(16) uint16_t qs[G][DH];
  __shared__ float red[2][4][G];
  __shared__ int last_flag;

  int b, hg, s;
  decode_work_item(a.B, a.H / G, a.nsplit, b, hg, s);
  const int tid = threadIdx.x;
  const int h0 = hg * G, hk = h0 / (a.H / a.Hk);
  int n_keys = a.seqlens[b] + a.seqlen_add;
  n_keys = max(0, min(n_keys, a.S));
  int per = (n_keys + a.nsplit - 1) / a.nsplit;
  per = (per + KPB - 1) / KPB * KPB;
  const int k0 = min(s * per, n_keys);
  const int k1 = min(n_keys, k0 + per);

  if (tid < G * (DH / 2)) {
    const int g = tid / (DH / 2), d = tid % (DH / 2);
    const uint16_t* qp = a.q + (int64_t)b * a.sq_b + (int64_t)(h0 + g) * a.sq_h;
    float x0 = E::val(qp[d]), x1 = E::val(qp[d + DH / 2]);
    if (a.cos) {
      const int tp = min(max(a.seqlens[b], 0), a.rope_len - 1);
      const float c = E::val(a.cos[(int64_t)tp * (DH / 2) + d]);
      const float sn = E::val(a.sin[(int64_t)tp * (DH / 2) + d]);
      const float r0 = x0 * c - x1 * sn, r1 = x0 * sn + x1 * c;
      x0 = r0; x1 = r1;
    }
    qs[g][d] = (uint16_t)E::bits(x0);
    qs[g][d + DH / 2] = (uint16_t)E::bits(x1);
  }
  const int part = tid % LPK, slot = tid / LPK;
  const uint16_t* kbase = a.k_cache + (int64_t)b * a.sc_b + (int64_t)hk * a.sc_h + part * 8;
  const uint16_t* vbase = a.v_cache + (int64_t)b * a.sc_b + (int64_t)hk * a.sc_h + part * 8;

  float m_run[G], l_thr[G], acc[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m_run[g] = -INFINITY; l_thr[g] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[g][i] = 0.f;
  }
  int it = 0;
  for (int c0 = k0; c0 < k1; c0 += CH, ++it) {
    u32x4_t kv[U], vv[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int key = min(c0 + u * KPB + slot, k1 - 1);
      kv[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(kbase + (int64_t)key * a.sc_s));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int key = min(c0 + u * KPB + slot, k1 - 1);
      vv[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(vbase + (int64_t)key * a.sc_s));
    }
    if (it == 0) __syncthreads();  // qs ready
    float sc[G][U];
    const int rb = it & 1;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const u32x4_t qv = *reinterpret_cast<const u32x4_t*>(&qs[g][part * 8]);
      float lmax = -INFINITY;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        float d = E::dot8(kv[u], qv, 0.f);
        d += dpp_f32<0xB1>(d);
        d += dpp_f32<0x4E>(d);
        d += dpp_f32<0x141>(d);
        if (LPK == 16) d += dpp_f32<0x140>(d);
        sc[g][u] = (c0 + u * KPB + slot < k1) ? d * a.scale : -INFINITY;
        lmax = fmaxf(lmax, sc[g][u]);
      }
      lmax = wave_max(lmax);
      if ((tid & 63) == 0) red[rb][tid >> 6][g] = lmax;
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const float m_c = fmaxf(fmaxf(red[rb][0][g], red[rb][1][g]), fmaxf(red[rb][2][g], red[rb][3][g]));
      const float m_new = fmaxf(m_run[g], m_c);
      const float alpha = (m_run[g] == -INFINITY) ? 0.f : __expf(m_run[g] - m_new);
      float psum = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[g][i] *= alpha;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const float p = (sc[g][u] == -INFINITY) ? 0.f : __expf(sc[g][u] - m_new);
        psum += p;
        acc[g][0] += p * E::lo(vv[u].x); acc[g][1] += p * E::hi(vv[u].x);
        acc[g][2] += p * E::lo(vv[u].y); acc[g][3] += p * E::hi(vv[u].y);
        acc[g][4] += p * E::lo(vv[u].z); acc[g][5] += p * E::hi(vv[u].z);
        acc[g][6] += p * E::lo(vv[u].w); acc[g][7] += p * E::hi(vv[u].w);
      }
      l_thr[g] = l_thr[g] * alpha + (part == 0 ? psum : 0.f);
      m_run[g] = m_new;
    }
  }
  if (it == 0) __syncthreads();
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const int h = h0 + g;
    // fold the key slots and the per-thread sums of this head (the LDS block is free: the barriers below end every round)
#pragma unroll
    for (int i = 0; i < 8; ++i) accs[slot * DH + part * 8 + i] = acc[g][i];
    const float lw = wave_sum(l_thr[g]);
    __syncthreads();
    if ((tid & 63) == 0) red[0][tid >> 6][0] = lw;
    __syncthreads();
    const float l = (red[0][0][0] + red[0][1][0]) + (red[0][2][0] + red[0][3][0]);
    const float m = m_run[g];
    float o = 0.f;
    if (tid < DH) {
#pragma unroll 8
      for (int j = 0; j < KPB; ++j) o += accs[j * DH + tid];
    }
    uint16_t* outp = a.out + (int64_t)b * a.so_b + (int64_t)h * a.so_h;
    if (a.nsplit == 1) {
      if (tid < DH) outp[tid] = (uint16_t)E::bits(l > 0.f ? o / l : 0.f);
      __syncthreads();                             // accs and red are read out before the next head refills them
      continue;
    }
    float* part_ws = a.ws_part + ((int64_t)(b * a.H + h) * a.nsplit) * (DH + 2);
    float* mine = part_ws + (int64_t)s * (DH + 2);
    if (tid < DH) st_agent(mine + tid, o);
    if (tid == 0) { st_agent(mine + DH, m); st_agent(mine + DH + 1, l); }
    wait_stores_acked();
    __syncthreads();
    if (tid == 0) {
      const int old = __hip_atomic_fetch_add(&a.ws_count[b * a.H + h], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      last_flag = (old == a.nsplit - 1);
    }
    __syncthreads();
    const bool last = last_flag != 0;
    if (last) {
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
      if (tid < DH) {
        constexpr int SU = 8;
        float M = -INFINITY;
        for (int i0 = 0; i0 < a.nsplit; i0 += SU) {
          float mi[SU];
#pragma unroll
          for (int u = 0; u < SU; ++u) mi[u] = ld_agent(part_ws + (int64_t)min(i0 + u, a.nsplit - 1) * (DH + 2) + DH);
#pragma unroll
          for (int u = 0; u < SU; ++u) M = fmaxf(M, mi[u]);
        }
        float num = 0.f, den = 0.f;
        for (int i0 = 0; i0 < a.nsplit; i0 += SU) {
          float mi[SU], oi[SU], li[SU];
#pragma unroll
          for (int u = 0; u < SU; ++u) {
            const float* pw = part_ws + (int64_t)min(i0 + u, a.nsplit - 1) * (DH + 2);
            mi[u] = ld_agent(pw + DH);
            oi[u] = ld_agent(pw + tid);
            li[u] = ld_agent(pw + DH + 1);
          }
#pragma unroll
          for (int u = 0; u < SU; ++u) {
            const float w = (i0 + u >= a.nsplit || mi[u] == -INFINITY) ? 0.f : __expf(mi[u] - M);
            num += w * oi[u];
            den += w * li[u];
          }
        }
        outp[tid] = (uint16_t)E::bits(den > 0.f ? num / den : 0.f);
      }
      if (tid == 0) __hip_atomic_store(&a.ws_count[b * a.H + h], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();                               // last_flag, accs and red are read out before the next head reuses them
  }
}

// rotate k_new at position seqlens[b] (fp32 math, one rounding) and write k/v into the caches
template <int DT>
__global__ __launch_bounds__(256) void kv_append_kernel(KvAppendArgs a) {
  typedef E16<DT> E;
  const int half = a.Dh >> 1;
  const int total = a.B * a.Hk * half;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < total; i += gridDim.x * blockDim.x) {
    const int d = i % half, hk = (i / half) % a.Hk, b = i / (half * a.Hk);
    const int pos = a.seqlens[b];
    if (pos < 0 || pos >= a.S) continue;
    const uint16_t* kp = a.k_new + (int64_t)b * a.sk_b + (int64_t)hk * a.sk_h;
    const uint16_t* vp = a.v_new + (int64_t)b * a.sv_b + (int64_t)hk * a.sv_h;
    float x0 = E::val(kp[d]), x1 = E::val(kp[d + half]);
    if (a.cos) {
      const int tp = min(pos, a.rope_len - 1);
      const float c = E::val(a.cos[(int64_t)tp * half + d]);
      const float s = E::val(a.sin[(int64_t)tp * half + d]);
      const float r0 = x0 * c - x1 * s, r1 = x0 * s + x1 * c;
      x0 = r0; x1 = r1;
    }
    const int64_t off = (int64_t)b * a.sc_b + (int64_t)pos * a.sc_s + (int64_t)hk * a.sc_h;
    a.k_cache[off + d] = (uint16_t)E::bits(x0);
    a.k_cache[off + d + half] = (uint16_t)E::bits(x1);
    a.v_cache[off + d] = vp[d];
    a.v_cache[off + d + half] = vp[d + half];
  }
}

size_t attn_decode_ws_floats(int B, int H, int nsplit, int Dh) { return (size_t)B * H * nsplit * (Dh + 2); }

template <int DT>
static void launch_attn_decode_t(const AttnDecodeArgs& a, int G, hipStream_t st) {
  dim3 grid(a.B * (a.H / G) * a.nsplit);
  if (G == 4) hipLaunchKernelGGL((attn_decode_gqa_kernel<DT, 128, 8, 4>), grid, dim3(kAttnThreads), 0, st, a);
  else if (G == 2) hipLaunchKernelGGL((attn_decode_gqa_kernel<DT, 128, 8, 2>), grid, dim3(kAttnThreads), 0, st, a);
  else if (a.Dh == 128) hipLaunchKernelGGL((attn_decode_kernel<DT, 128, 8>), grid, dim3(kAttnThreads), 0, st, a);
  else hipLaunchKernelGGL((attn_decode_kernel<DT, 64, 4>), grid, dim3(kAttnThreads), 0, st, a);
}

int launch_attn_decode(const AttnDecodeArgs& a, hipStream_t st) {
  if (a.dt != 0 && a.dt != 1) { set_last_error("fsvd_attn_decode_densekv: dtype code %d (bf16 = 0 and fp16 = 1 are served)", a.dt); return kErrBadDtype; }
  if (a.B <= 0 || a.H <= 0 || a.Hk <= 0 || a.H % a.Hk != 0 || a.S <= 0 || a.nsplit <= 0) {
    set_last_error("fsvd_attn_decode_densekv: bad shape B=%d H=%d Hk=%d S=%d nsplit=%d", a.B, a.H, a.Hk, a.S, a.nsplit);
    return kErrBadShape;
  }
  if (a.Dh != 64 && a.Dh != 128) { set_last_error("fsvd_attn_decode_densekv: head_dim %d not in {64,128}", a.Dh); return kErrBadShape; }
  const int kpb = kAttnThreads / (a.Dh / 8);
  const int per = ((a.S + a.nsplit - 1) / a.nsplit + kpb - 1) / kpb * kpb;
  if (per > kMaxKeysPerSplit) {
    set_last_error("fsvd_attn_decode_densekv: %d keys per split exceeds %d; raise nsplit", per, kMaxKeysPerSplit);
    return kErrBadShape;
  }
  if ((a.sc_s % 8) || (a.sc_h % 8) || (a.sc_b % 8) || (reinterpret_cast<uintptr_t>(a.k_cache) & 15) ||
      (reinterpret_cast<uintptr_t>(a.v_cache) & 15)) {
    set_last_error("fsvd_attn_decode_densekv: cache strides/pointers must be 16-byte aligned");
    return kErrBadAlign;
  }
  if (a.nsplit > 1 && (!a.ws_part || !a.ws_count)) { set_last_error("fsvd_attn_decode_densekv: workspace missing"); return kErrWorkspace; }
  // grouped-query caches with enough work to fill the chip four (two) query heads at a time: the kv rows are read once
  // per group of query heads
  const int rep = a.H / a.Hk;
  int G = 1;
  if (a.Dh == 128) {
    if (rep % 4 == 0 && (int64_t)a.B * (a.H / 4) * a.nsplit >= 512) G = 4;
    else if (rep % 2 == 0 && (int64_t)a.B * (a.H / 2) * a.nsplit >= 512) G = 2;
  }
  if (a.dt == 1) launch_attn_decode_t<1>(a, G, st);
  else launch_attn_decode_t<0>(a, G, st);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("fsvd_attn_decode_densekv: launch failed: %s", hipGetErrorString(e)); return kErrLaunch; }
  return kOk;
}

int launch_kv_append(const KvAppendArgs& a, hipStream_t st) {
  if (a.B <= 0 || a.Hk <= 0 || a.Dh <= 0 || (a.Dh & 1) || a.S <= 0) { set_last_error("fsvd_kv_append: bad shape"); return kErrBadShape; }
  const int total = a.B * a.Hk * (a.Dh / 2);
  if (a.dt != 0 && a.dt != 1) { set_last_error("fsvd_kv_append: dtype code %d (bf16 = 0 and fp16 = 1 are served)", a.dt); return kErrBadDtype; }
  if (a.dt == 1) hipLaunchKernelGGL(kv_append_kernel<1>, dim3((total + 255) / 256), dim3(256), 0, st, a);
  else hipLaunchKernelGGL(kv_append_kernel<0>, dim3((total + 255) / 256), dim3(256), 0, st, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("fsvd_kv_append: launch failed: %s", hipGetErrorString(e)); return kErrLaunch; }
  return kOk;
}

}  // namespace fsvd
