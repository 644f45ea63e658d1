// Full-sequence (prefill) side of the low-rank RoPE attention, split the way a 288 GB part wants it:
//
//  1. lowrank_expand_kernel — Y = P @ u^T on the matrix cores for all tokens at once, with the head
//     epilogue fused: bias, rotate-half RoPE at the token's absolute position, and a strided store
//     straight into its destination (the query buffer [B,M,H,dh], or the dense KV cache rows
//     [B,S,Hk,dh] the decode kernels read later).  Both MFMA operands are contiguous along the rank
//     axis (P rows, nn.Linear-layout u rows), so they are plain 16-byte global loads in the
//     instruction's native lane layout; a wave owns 32 tokens x 128 head columns (16 accumulator
//     tiles) and d / d+64 of a head sit in the same lane, which keeps the rotation register-local.
//     K and V are rebuilt exactly once per token (the reference's fused kernel rebuilds every key
//     tile once per query tile to avoid the HBM round trip; with 288 GB that trade goes the other way).
//
//  2. attn_prefill_kernel — causal flash attention over the rotated q and the cache rows: S = Q K^T
//     and O += P V on MFMA 16x16x32 bf16, online softmax in fp32 on the accumulator layout, P passed
//     through LDS (as a bf16 high part plus a bf16 residual) to become an A operand, V tile transposed through LDS to become a B operand.
//     Key padding mask, additive mask and "fully masked row -> 0" follow the reference kernel.
#include "common.hpp"
#include "kernels.hpp"

namespace fsvd {

constexpr int kPfThreads = 256;

// eight elements as a matrix-core operand (F = the element type's fragment)
template <class F>
__device__ __forceinline__ F pf_ld(const uint16_t* p) {
  return __builtin_bit_cast(F, *reinterpret_cast<const u32x4_t*>(p));
}
template <class F>
__device__ __forceinline__ F pf_zero() { return __builtin_bit_cast(F, u32x4_t{0u, 0u, 0u, 0u}); }

// ---------------------------------------------------------------------------------------------
// 1. Y[token, head, :] = epilogue( P[token, (head), :] @ u[head*128 + :, :]^T )
//    grid (ceil(T/128), heads), 4 waves x 32 tokens
// ---------------------------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(kPfThreads) void lowrank_expand_kernel(ExpandArgs a) {
  typedef E16<DT> E;
  typedef typename E::frag_t frag_t;
  constexpr int DH = 128, NT = 8, HALF = 64;
  const int head = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lr = lane & 15, lg = lane >> 4;
  const int T = a.B * a.M;
  const int row0 = blockIdx.x * 128 + wave * 32;
  if (row0 >= T) return;

  const uint16_t* arow[2];
#pragma unroll
  for (int mi = 0; mi < 2; ++mi) {
    const int r = min(row0 + mi * 16 + lr, T - 1);
    const int b = r / a.M, m = r % a.M;
    arow[mi] = a.p + (int64_t)b * a.sp_b + (int64_t)m * a.sp_m + (int64_t)head * a.sp_h + lg * 8;
  }
  const uint16_t* brow = a.u + (int64_t)(head * DH + lr) * a.ldu + lg * 8;

  f32x4_t acc[2][NT];
#pragma unroll
  for (int mi = 0; mi < 2; ++mi)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[mi][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
  for (int r0 = 0; r0 < a.R; r0 += 32) {
    const bool in = r0 + lg * 8 < a.R;
    frag_t af[2], bf[NT];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) af[mi] = in ? pf_ld<frag_t>(arow[mi] + r0) : pf_zero<frag_t>();
#pragma unroll
    for (int t = 0; t < NT; ++t) bf[t] = in ? pf_ld<frag_t>(brow + (int64_t)t * 16 * a.ldu + r0) : pf_zero<frag_t>();
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[mi][t] = E::mfma(af[mi], bf[t], acc[mi][t]);
  }

  // epilogue on the accumulator layout: lane holds rows lg*4+i, column t*16+lr of each tile
#pragma unroll
  for (int mi = 0; mi < 2; ++mi)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = row0 + mi * 16 + lg * 4 + i;
      if (r >= T) continue;
      const int b = r / a.M, m = r % a.M;
      const int pos = (a.positions ? a.positions[b] : 0) + m;
      float x[NT];
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        float v = acc[mi][t][i];
        if (a.bias) v += E::val(a.bias[head * DH + t * 16 + lr]);
        x[t] = E::rnd(v);                       // the projection's own rounding point
      }
      if (a.cos) {
        // eager bf16 arithmetic: x0*c - x1*s and x1*c + x0*s, one rounding per op
        const int tp = min(max(pos, 0), a.rope_len - 1);
#pragma unroll
        for (int t = 0; t < NT / 2; ++t) {
          const float c = E::val(a.cos[(int64_t)tp * HALF + t * 16 + lr]);
          const float s = E::val(a.sin[(int64_t)tp * HALF + t * 16 + lr]);
          const float x0 = x[t], x1 = x[t + NT / 2];
          x[t] = E::rnd(E::rnd(x0 * c) - E::rnd(x1 * s));
          x[t + NT / 2] = E::rnd(E::rnd(x1 * c) + E::rnd(x0 * s));
        }
      }
      const int slot = a.dst_by_position ? pos : m;
      if (slot < 0 || slot >= a.dst_rows) continue;   // outside the destination: dropped
      uint16_t* dst = a.y + (int64_t)b * a.sy_b + (int64_t)slot * a.sy_m + (int64_t)head * a.sy_h;
#pragma unroll
      for (int t = 0; t < NT; ++t) dst[t * 16 + lr] = (uint16_t)E::bits(x[t]);
    }
}

// ---------------------------------------------------------------------------------------------
// 2. causal flash attention, head_dim 128, 64 queries per workgroup (16 per wave), 64-key tiles
// ---------------------------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(kPfThreads) void attn_prefill_kernel(PrefillAttnArgs a) {
  typedef E16<DT> E;
  typedef typename E::frag_t frag_t;
  constexpr int DH = 128, BN = 64, PSTR = BN + 8, VSTR = BN + 8;
  __shared__ __align__(16) uint16_t Ps[4][16][PSTR];    // softmax weights, bf16 high part
  __shared__ __align__(16) uint16_t Pl[4][16][PSTR];    // and the bf16 residual, so that P carries ~16 mantissa bits
  __shared__ __align__(16) uint16_t Vt[DH][VSTR];

  const int mt = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int hk = h / (a.H / a.Hk);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lr = lane & 15, lg = lane >> 4;
  const int q0 = a.q_pos0 ? a.q_pos0[b] : 0;          // absolute position of query row 0
  const int m_base = mt * 64 + wave * 16;             // first query row of this wave
  const int n_keys_all = max(1, min(q0 + a.M, a.S));  // keys that exist once the block is appended

  // Q fragments (A operand): row m_base+lr, d = step*32 + lg*8
  frag_t qf[4];
  {
    const int m = min(m_base + lr, a.M - 1);
    const uint16_t* qp = a.q + (int64_t)b * a.sq_b + (int64_t)m * a.sq_m + (int64_t)h * a.sq_h + lg * 8;
#pragma unroll
    for (int st = 0; st < 4; ++st) qf[st] = pf_ld<frag_t>(qp + st * 32);
  }
  float m_run[4], l_run[4];
  f32x4_t o[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) { m_run[i] = -INFINITY; l_run[i] = 0.f; }
#pragma unroll
  for (int t = 0; t < 8; ++t) o[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // last key any row of this workgroup may see (causal): position of its last valid query
  const int last_m = min(mt * 64 + 63, a.M - 1);
  const int k_end = a.causal ? min(n_keys_all, q0 + last_m + 1) : n_keys_all;
  const uint16_t* kb = a.k + (int64_t)b * a.sk_b + (int64_t)hk * a.sk_h;
  const uint16_t* vb = a.v + (int64_t)b * a.sk_b + (int64_t)hk * a.sk_h;

  for (int n0 = 0; n0 < k_end; n0 += BN) {
    // ---- stage V tile transposed: thread -> key n0 + tid/16 (+16 per pass), d0 = (tid%16)*8
    __syncthreads();   // previous tile's Vt / Ps fully consumed
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
      const int kk = pass * 16 + (tid >> 4);
      const int key = min(n0 + kk, n_keys_all - 1);
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(vb + (int64_t)key * a.sk_s + (tid & 15) * 8);
      const int d0 = (tid & 15) * 8;
      Vt[d0 + 0][kk] = (uint16_t)(v.x & 0xffff); Vt[d0 + 1][kk] = (uint16_t)(v.x >> 16);
      Vt[d0 + 2][kk] = (uint16_t)(v.y & 0xffff); Vt[d0 + 3][kk] = (uint16_t)(v.y >> 16);
      Vt[d0 + 4][kk] = (uint16_t)(v.z & 0xffff); Vt[d0 + 5][kk] = (uint16_t)(v.z >> 16);
      Vt[d0 + 6][kk] = (uint16_t)(v.w & 0xffff); Vt[d0 + 7][kk] = (uint16_t)(v.w >> 16);
    }
    // ---- S = Q K^T for 16 rows x 64 keys (4 tiles); K rows are B operands straight from memory
    f32x4_t s[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      s[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      const int key = min(n0 + j * 16 + lr, n_keys_all - 1);
      const uint16_t* kp = kb + (int64_t)key * a.sk_s + lg * 8;
#pragma unroll
      for (int st = 0; st < 4; ++st) s[j] = E::mfma(qf[st], pf_ld<frag_t>(kp + st * 32), s[j]);
    }
    // ---- masks + online softmax on the accumulator layout (rows lg*4+i, key column j*16+lr)
    float p[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m_base + lg * 4 + i;
      const int qpos = q0 + m;
      float rmax = -INFINITY;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int key = n0 + j * 16 + lr;
        float v = s[j][i];
        bool ok = key < n_keys_all && m < a.M;
        if (a.causal) ok = ok && key <= qpos;
        v = ok ? v * a.scale : -INFINITY;            // mask first, then scale, as the reference kernel
        if (ok && a.pad_mask) ok = a.pad_mask[(int64_t)b * a.spm_b + key] != 0;
        if (!ok) v = -INFINITY;
        if (ok && a.add_mask) v += a.add_mask[(int64_t)b * a.sam_b + (int64_t)m * a.sam_q + key];
        p[j][i] = v;
        rmax = fmaxf(rmax, v);
      }
      rmax = row16_max(rmax);
      const float m_new = fmaxf(m_run[i], rmax);
      const float alpha = (m_run[i] == -INFINITY) ? 0.f : __expf(m_run[i] - m_new);
      float rsum = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float e = (p[j][i] == -INFINITY || m_new == -INFINITY) ? 0.f : __expf(p[j][i] - m_new);
        p[j][i] = e;
        rsum += e;
      }
      rsum = row16_sum(rsum);
      l_run[i] = l_run[i] * alpha + rsum;
      m_run[i] = m_new;
#pragma unroll
      for (int t = 0; t < 8; ++t) o[t][i] *= alpha;
    }
    // ---- P (bf16) to LDS in row-major so that it can be re-read as an A operand
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t hi = E::bits(p[j][i]);
        Ps[wave][lg * 4 + i][j * 16 + lr] = (uint16_t)hi;
        Pl[wave][lg * 4 + i][j * 16 + lr] = (uint16_t)E::bits(p[j][i] - E::val(hi));
      }
    __syncthreads();   // Vt and Ps visible
    // ---- O += P V : A = Ps[row lr][keys st*32 + lg*8 ..], B = Vt[d = t*16+lr][keys st*32 + lg*8 ..]
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const frag_t pa = pf_ld<frag_t>(&Ps[wave][lr][st * 32 + lg * 8]);
      const frag_t pb = pf_ld<frag_t>(&Pl[wave][lr][st * 32 + lg * 8]);
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const frag_t vf = pf_ld<frag_t>(&Vt[t * 16 + lr][st * 32 + lg * 8]);
        o[t] = E::mfma(pa, vf, o[t]);
        o[t] = E::mfma(pb, vf, o[t]);
      }
    }
  }

  // ---- normalise and store; rows with no visible key give 0
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m_base + lg * 4 + i;
    if (m >= a.M) continue;
    const float inv = l_run[i] > 0.f ? 1.0f / l_run[i] : 0.f;
    uint16_t* op = a.out + (int64_t)b * a.so_b + (int64_t)m * a.so_m + (int64_t)h * a.so_h;
#pragma unroll
    for (int t = 0; t < 8; ++t) op[t * 16 + lr] = (uint16_t)E::bits(o[t][i] * inv);
  }
}

// ---------------------------------------------------------------------------------------------
// 2b. the same attention for long prompts: 64 or 128 queries per workgroup (16 MI per wave), K and V tiles shared
//     through LDS.  With every wave fetching its own K fragments a 64-key tile costs 80 KB of L2 traffic per 64
//     queries and the kernel is bound by L2 requests; here a tile is read ONCE per workgroup, coalesced, one tile
//     ahead into registers, and written to LDS (K row-major with a padded stride, V transposed: four adjacent keys
//     per 8-byte write, rows of 128 bytes whose 16-byte pieces are XOR-ed with (d / 2 % 8) ^ (d / 8 % 8): the 16-byte
//     fragment reads — served 16 lanes a cycle, lanes 0-3, 12-15, 20-27 / 4-11, 16-19, 28-31 of a half wave — and the
//     8-byte transposing writes, 8 lanes a cycle, then both touch every bank once; found by enumeration).
//
//     Scores are computed TRANSPOSED, S^T = K Q^T: an accumulator lane then holds four consecutive keys of ONE query
//     (column lr), so the softmax statistics are one value per lane and query block, and the eight softmax weights a
//     lane owns in two 16-key blocks are exactly one B-operand fragment of O^T = V^T P^T — P never goes through LDS.
//     The price is a key order inside every 32 keys that the V tile has to follow: MFMA k-slot (lg, e) holds key
//     16 (e / 4) + 4 lg + e % 4, so V^T is stored with key offset ko at column 8 (ko % 16 / 4) + 4 (ko / 16) + ko % 4.
//     P is a bf16 high part plus a bf16 residual (two products per fragment) so that it carries ~16 mantissa bits.
// ---------------------------------------------------------------------------------------------
// NG = 2: eight waves; waves 4-7 are a second group with K / V tiles of its own that takes every other key tile, and the
// two groups' running statistics and outputs are merged through LDS at the end — for prompts whose (query tile, head)
// pairs number no more than the compute units, where a workgroup alone on its compute unit walks its key tiles with
// one wave per SIMD and waits out every load and barrier.
template <int DT, int MI, int NG>
__global__ __launch_bounds__(kPfThreads * NG, NG == 1 ? 2 : 1) void attn_prefill_wide_kernel(PrefillAttnArgs a) {
  typedef E16<DT> E;
  typedef typename E::frag_t frag_t;
  constexpr int DH = 128, BN = 64, QW = 16 * MI, BM = 4 * QW, VSTR = BN;
  // K rows of 288 bytes: a 16-byte LDS read is served 16 lanes a cycle (lanes 0-3, 12-15, 20-27 / 4-11, 16-19, 28-31 of a
  // half wave); rows 16 r apart with r odd multiples of 32 bytes give those lanes 16 different bank groups
  constexpr int KSTR = DH + 16;
  extern __shared__ __align__(16) unsigned char pw_smem[];
  constexpr int kGroupBytes = BN * KSTR * 2 + DH * VSTR * 2;
  const int grp = NG == 1 ? 0 : (int)(threadIdx.x >> 8);
  unsigned char* gsm = pw_smem + (size_t)grp * kGroupBytes;
  uint16_t (*Ks)[KSTR] = reinterpret_cast<uint16_t (*)[KSTR]>(gsm);                                   // [BN][KSTR]
  uint16_t (*Vt)[VSTR] = reinterpret_cast<uint16_t (*)[VSTR]>(gsm + (size_t)BN * KSTR * 2);            // [DH][VSTR]

  // the query tiles of a head (and the heads of a kv head) run on one XCD, so its K and V come out of one L2; under
  // a causal mask the last tiles, which see the most keys, start first
  const int MT = gridDim.x;
  const int t = xcd_run_index(blockIdx.x + MT * (blockIdx.y + gridDim.y * blockIdx.z), MT * gridDim.y * gridDim.z);
  const int mt = a.causal ? MT - 1 - t % MT : t % MT, h = (t / MT) % (int)gridDim.y, b = t / (MT * (int)gridDim.y);
  const int hk = h / (a.H / a.Hk);
  const int tid = threadIdx.x & 255, lane = tid & 63, wave = tid >> 6;   // thread and wave within the group
  const int lr = lane & 15, lg = lane >> 4;
  const int q0 = a.q_pos0 ? a.q_pos0[b] : 0;
  const int m_base = mt * BM + wave * QW;
  const int n_keys_all = max(1, min(q0 + a.M, a.S));

  frag_t qf[MI][4];
#pragma unroll
  for (int mi = 0; mi < MI; ++mi) {
    const int m = min(m_base + mi * 16 + lr, a.M - 1);
    const uint16_t* qp = a.q + (int64_t)b * a.sq_b + (int64_t)m * a.sq_m + (int64_t)h * a.sq_h + lg * 8;
#pragma unroll
    for (int st = 0; st < 4; ++st) qf[mi][st] = pf_ld<frag_t>(qp + st * 32);
  }
  float m_run[MI], l_run[MI];          // statistics of query m_base + 16 mi + lr (the same in the four lanes lg of a column)
  f32x4_t o[MI][8];                    // O^T: tile t, element i = dimension 16 t + 4 lg + i of that query
#pragma unroll
  for (int mi = 0; mi < MI; ++mi) {
    m_run[mi] = -INFINITY; l_run[mi] = 0.f;
#pragma unroll
    for (int t = 0; t < 8; ++t) o[mi][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  const int last_m = min(mt * BM + BM - 1, a.M - 1);
  const int k_end = a.causal ? min(n_keys_all, q0 + last_m + 1) : n_keys_all;
  // last key this wave's rows may see: tiles past it are skipped by the wave (it still takes part in the staging)
  const int wave_end = a.causal ? min(n_keys_all, q0 + min(m_base + QW - 1, a.M - 1) + 1) : n_keys_all;
  const bool rows_ragged = m_base + QW > a.M;
  const uint16_t* kb = a.k + (int64_t)b * a.sk_b + (int64_t)hk * a.sk_h;
  const uint16_t* vb = a.v + (int64_t)b * a.sk_b + (int64_t)hk * a.sk_h;

  // staging roles: 16 lanes cover one 256-byte row; K: rows tid/16 + 16 j; V: the four adjacent keys 4 (tid/16) + j
  const int srow = tid >> 4, d0 = (tid & 15) * 8;
  // column of this thread's four keys in the permuted order of V^T (see above), before the bank swizzle
  const int vko = (srow * 4) & 31;
  const int vcol = ((srow * 4) & 32) + 8 * ((vko & 15) >> 2) + 4 * (vko >> 4);
  u32x4_t kreg[4], vreg[4];
  // the padding-mask bytes of a key tile travel with it: requested with the tile (threads 0-63, one key each), parked in
  // LDS beside it, read from there four keys at a time (read from memory where they apply, each under its own test,
  // they are sixteen memory round trips in a row per query block and tile)
  __shared__ __align__(16) uint8_t pms[NG][BN];
  uint8_t pmreg = 1;
  auto request = [&](int n0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int kkey = min(n0 + srow + 16 * j, n_keys_all - 1), vkey = min(n0 + srow * 4 + j, n_keys_all - 1);
      kreg[j] = *reinterpret_cast<const u32x4_t*>(kb + (int64_t)kkey * a.sk_s + d0);
      vreg[j] = *reinterpret_cast<const u32x4_t*>(vb + (int64_t)vkey * a.sk_s + d0);
    }
    if (a.pad_mask && tid < BN) pmreg = a.pad_mask[(int64_t)b * a.spm_b + min(n0 + tid, n_keys_all - 1)];
  };
  if (grp * BN < k_end) request(grp * BN);

  for (int n00 = 0; n00 < k_end; n00 += NG * BN) {
    const int n0 = n00 + grp * BN;
    const bool live = n0 < k_end;       // the second group may have no tile in the last round; it still meets the barriers
    __syncthreads();   // the previous tile's Ks / Vt are consumed
    if (live) {
    if (a.pad_mask && tid < BN) pms[grp][tid] = pmreg;
#pragma unroll
    for (int j = 0; j < 4; ++j) *reinterpret_cast<u32x4_t*>(&Ks[srow + 16 * j][d0]) = kreg[j];
    {
      const uint32_t w[4][4] = {{vreg[0].x, vreg[0].y, vreg[0].z, vreg[0].w}, {vreg[1].x, vreg[1].y, vreg[1].z, vreg[1].w},
                                {vreg[2].x, vreg[2].y, vreg[2].z, vreg[2].w}, {vreg[3].x, vreg[3].y, vreg[3].z, vreg[3].w}};
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        u32x2_t lo, hi;   // dimensions d0 + 2c (low halves) and d0 + 2c + 1 (high halves) of the four keys
        lo.x = (w[0][c] & 0xffffu) | (w[1][c] << 16);
        lo.y = (w[2][c] & 0xffffu) | (w[3][c] << 16);
        hi.x = (w[0][c] >> 16) | (w[1][c] & 0xffff0000u);
        hi.y = (w[2][c] >> 16) | (w[3][c] & 0xffff0000u);
        // rows d0 + 2c and d0 + 2c + 1 share the swizzle term (row / 2 % 8) ^ (row / 8 % 8)
        const int col = vcol ^ (8 * (((((tid & 1) << 2) + c) ^ (tid & 7))));
        *reinterpret_cast<u32x2_t*>(&Vt[d0 + 2 * c][col]) = lo;
        *reinterpret_cast<u32x2_t*>(&Vt[d0 + 2 * c + 1][col]) = hi;
      }
    }
    }
    __syncthreads();   // tile visible
    if (n0 + NG * BN < k_end) request(n0 + NG * BN);
    if (!live || n0 >= wave_end) continue;   // nothing this wave's rows may see (wave-uniform)

    // ---- S^T = K Q^T for 64 keys x 16 MI queries: block j, element i = key n0 + 16 j + 4 lg + i, query column lr
    f32x4_t sacc[MI][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      frag_t kf[4];
#pragma unroll
      for (int st = 0; st < 4; ++st) kf[st] = pf_ld<frag_t>(&Ks[j * 16 + lr][st * 32 + lg * 8]);
#pragma unroll
      for (int mi = 0; mi < MI; ++mi) {
        sacc[mi][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int st = 0; st < 4; ++st) sacc[mi][j] = E::mfma(kf[st], qf[mi][st], sacc[mi][j]);
      }
    }
    // ---- masks + online softmax, one query per lane and block; tiles that need no mask take the short way
    const bool plain = !a.pad_mask && !a.add_mask && !rows_ragged && n0 + BN <= n_keys_all &&
                       (!a.causal || n0 + BN - 1 <= q0 + m_base);
    frag_t ph[MI][2], pl[MI][2];     // P^T fragments (high part, residual) of the two 32-key steps
    uint32_t pmw[4] = {0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u};   // mask bytes of keys n0 + 16 j + 4 lg + (0..3)
    if (!plain && a.pad_mask) {
#pragma unroll
      for (int j = 0; j < 4; ++j) pmw[j] = *reinterpret_cast<const uint32_t*>(&pms[grp][j * 16 + lg * 4]);
    }
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
      const int m = m_base + mi * 16 + lr;
      const int qpos = q0 + m;
      float mx = -INFINITY;
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v = sacc[mi][j][i] * a.scale;
          if (!plain) {
            const int key = n0 + j * 16 + lg * 4 + i;
            bool ok = key < n_keys_all && m < a.M;
            if (a.causal) ok = ok && key <= qpos;
            ok = ok && ((pmw[j] >> (8 * i)) & 0xffu) != 0;
            if (!ok) v = -INFINITY;                    // mask first, then the additive term, as the reference kernel
            else if (a.add_mask) v += a.add_mask[(int64_t)b * a.sam_b + (int64_t)m * a.sam_q + key];
          }
          sacc[mi][j][i] = v;
          mx = fmaxf(mx, v);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16));
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      const float m_new = fmaxf(m_run[mi], mx);
      const float alpha = (m_run[mi] == -INFINITY) ? 0.f : __expf(m_run[mi] - m_new);
      float rsum = 0.f;
      float e[4][4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float v = sacc[mi][j][i];
          e[j][i] = (v == -INFINITY || m_new == -INFINITY) ? 0.f : __expf(v - m_new);
          rsum += e[j][i];
        }
      rsum += __shfl_xor(rsum, 16);
      rsum += __shfl_xor(rsum, 32);
      l_run[mi] = l_run[mi] * alpha + rsum;
      m_run[mi] = m_new;
#pragma unroll
      for (int t = 0; t < 8; ++t) o[mi][t] *= alpha;
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        uint32_t hw[4], lw[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {                  // k-slots 2c, 2c + 1: block 2 st + c / 2, elements 2 (c % 2), + 1
          const float x0 = e[2 * st + (c >> 1)][2 * (c & 1)], x1 = e[2 * st + (c >> 1)][2 * (c & 1) + 1];
          const uint32_t h0 = E::bits(x0), h1 = E::bits(x1);
          hw[c] = h0 | (h1 << 16);
          lw[c] = E::bits(x0 - E::val(h0)) | (E::bits(x1 - E::val(h1)) << 16);
        }
        ph[mi][st] = __builtin_bit_cast(frag_t, u32x4_t{hw[0], hw[1], hw[2], hw[3]});
        pl[mi][st] = __builtin_bit_cast(frag_t, u32x4_t{lw[0], lw[1], lw[2], lw[3]});
      }
    }
    // ---- O^T += V^T P^T : A = Vt rows (dimension 16 t + lr; keys in the permuted order), B = P^T fragments
#pragma unroll
    for (int st = 0; st < 2; ++st) {
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const frag_t vf = pf_ld<frag_t>(&Vt[t * 16 + lr][(st * 32 + lg * 8) ^ (8 * ((lr >> 1) ^ ((2 * t + (lr >> 3)) & 7)))]);
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
          o[mi][t] = E::mfma(vf, ph[mi][st], o[mi][t]);
          o[mi][t] = E::mfma(vf, pl[mi][st], o[mi][t]);
        }
      }
    }
  }

  if (NG == 2) {
    // merge the two groups: (m, l, O) of group 1 through LDS (word-major, one 16-byte word per lane and slot)
    f32x4_t* mb = reinterpret_cast<f32x4_t*>(pw_smem);
    __syncthreads();                   // both groups are done with their K / V tiles
    if (grp == 1) {
#pragma unroll
      for (int mi = 0; mi < MI; ++mi) {
        mb[(mi * 9) * 256 + tid] = f32x4_t{m_run[mi], l_run[mi], 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < 8; ++t) mb[(mi * 9 + 1 + t) * 256 + tid] = o[mi][t];
      }
    }
    __syncthreads();
    if (grp == 1) return;
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
      const f32x4_t st = mb[(mi * 9) * 256 + tid];
      const float m1 = st[0], l1 = st[1];
      const float m = fmaxf(m_run[mi], m1);
      const float a0 = m_run[mi] == -INFINITY ? 0.f : __expf(m_run[mi] - m), a1 = m1 == -INFINITY ? 0.f : __expf(m1 - m);
      l_run[mi] = l_run[mi] * a0 + l1 * a1;
#pragma unroll
      for (int t = 0; t < 8; ++t) o[mi][t] = o[mi][t] * a0 + mb[(mi * 9 + 1 + t) * 256 + tid] * a1;
    }
  }
  // ---- normalise and store (four consecutive dimensions per lane and tile); rows with no visible key give 0
#pragma unroll
  for (int mi = 0; mi < MI; ++mi) {
    const int m = m_base + mi * 16 + lr;
    if (m >= a.M) continue;
    const float inv = l_run[mi] > 0.f ? 1.0f / l_run[mi] : 0.f;
    uint16_t* op = a.out + (int64_t)b * a.so_b + (int64_t)m * a.so_m + (int64_t)h * a.so_h + lg * 4;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      u32x2_t w;
      w.x = E::bits(o[mi][t][0] * inv) | (E::bits(o[mi][t][1] * inv) << 16);
      w.y = E::bits(o[mi][t][2] * inv) | (E::bits(o[mi][t][3] * inv) << 16);
      *reinterpret_cast<u32x2_t*>(op + t * 16) = w;
    }
  }
}

int launch_expand(const ExpandArgs& a, hipStream_t st) {
  const char* fn = "fsvd_lowrank_expand_heads";
  if (a.dt != 0 && a.dt != 1) { set_last_error("%s: dtype code %d (bf16 = 0 and fp16 = 1 are served)", fn, a.dt); return kErrBadDtype; }
  if (a.B <= 0 || a.M <= 0 || a.heads <= 0 || a.R <= 0) { set_last_error("%s: empty shape", fn); return kErrBadShape; }
  if (a.Dh != 128) { set_last_error("%s: head_dim %d is not 128", fn, a.Dh); return kErrBadShape; }
  if (a.R % 8) { set_last_error("%s: rank %d is not a multiple of 8; pad the factors", fn, a.R); return kErrBadShape; }
  const auto mis = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) != 0; };
  if (mis(a.p) || mis(a.u) || (a.sp_b % 8) || (a.sp_m % 8) || (a.sp_h % 8) || (a.ldu % 8)) {
    set_last_error("%s: coefficient / factor pointers and strides must be 16-byte aligned", fn);
    return kErrBadAlign;
  }
  if (expand_tiles_apply(a)) return launch_expand_tiles(a, st);   // long prompts: the LDS-tiled kernel
  const int T = a.B * a.M;
  if (a.dt == 1) hipLaunchKernelGGL(lowrank_expand_kernel<1>, dim3((T + 127) / 128, a.heads), dim3(kPfThreads), 0, st, a);
  else hipLaunchKernelGGL(lowrank_expand_kernel<0>, dim3((T + 127) / 128, a.heads), dim3(kPfThreads), 0, st, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("%s: launch failed: %s", fn, hipGetErrorString(e)); return kErrLaunch; }
  return kOk;
}

template <int DT>
static int launch_prefill_attn_t(const PrefillAttnArgs& a, hipStream_t st) {
  const char* fn = "fsvd_attn_prefill";
  // the LDS-shared kernel stores four dimensions of a row with one 8-byte write
  const bool out8 = (reinterpret_cast<uintptr_t>(a.out) & 7) == 0 && (a.so_b % 4) == 0 && (a.so_m % 4) == 0 && (a.so_h % 4) == 0;
  if (a.M >= 128 && out8) {   // long prompts: 64 or 128 queries per workgroup, K / V tiles shared through LDS
    // 128 query rows per workgroup when that gives every compute unit work, else 64 (half the rows per wave)
    const bool wide = (int64_t)((a.M + 127) / 128) * a.H * a.B >= 384;
    const size_t lds = (size_t)64 * 144 * 2 + (size_t)128 * 64 * 2;
    // no more 64-row workgroups than ~1.25 per compute unit: two groups of waves share the key tiles of each
    const bool pair = !wide && (int64_t)((a.M + 63) / 64) * a.H * a.B <= 320;
    if (pair) {
      static bool granted = false;
      if (!granted) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_prefill_wide_kernel<DT, 1, 2>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)(2 * lds));
        if (e != hipSuccess) { set_last_error("%s: cannot reserve %zu bytes of LDS: %s", fn, 2 * lds, hipGetErrorString(e)); return kErrLaunch; }
        granted = true;
      }
      hipLaunchKernelGGL((attn_prefill_wide_kernel<DT, 1, 2>), dim3((a.M + 63) / 64, a.H, a.B), dim3(2 * kPfThreads), 2 * lds, st, a);
    } else if (wide) hipLaunchKernelGGL((attn_prefill_wide_kernel<DT, 2, 1>), dim3((a.M + 127) / 128, a.H, a.B), dim3(kPfThreads), lds, st, a);
    else hipLaunchKernelGGL((attn_prefill_wide_kernel<DT, 1, 1>), dim3((a.M + 63) / 64, a.H, a.B), dim3(kPfThreads), lds, st, a);
  } else {
    hipLaunchKernelGGL(attn_prefill_kernel<DT>, dim3((a.M + 63) / 64, a.H, a.B), dim3(kPfThreads), 0, st, a);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("%s: launch failed: %s", fn, hipGetErrorString(e)); return kErrLaunch; }
  return kOk;
}

int launch_prefill_attn(const PrefillAttnArgs& a, hipStream_t st) {
  const char* fn = "fsvd_attn_prefill";
  if (a.dt != 0 && a.dt != 1) { set_last_error("%s: dtype code %d (bf16 = 0 and fp16 = 1 are served)", fn, a.dt); return kErrBadDtype; }
  if (a.B <= 0 || a.M <= 0 || a.H <= 0 || a.Hk <= 0 || a.H % a.Hk) { set_last_error("%s: bad shape", fn); return kErrBadShape; }
  if (a.Dh != 128) { set_last_error("%s: head_dim %d is not 128", fn, a.Dh); return kErrBadShape; }
  const auto mis = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) != 0; };
  if (mis(a.q) || mis(a.k) || mis(a.v) || (a.sq_b % 8) || (a.sq_m % 8) || (a.sq_h % 8) || (a.sk_b % 8) || (a.sk_s % 8) || (a.sk_h % 8)) {
    set_last_error("%s: q / k / v pointers and strides must be 16-byte aligned", fn);
    return kErrBadAlign;
  }
  return a.dt == 1 ? launch_prefill_attn_t<1>(a, st) : launch_prefill_attn_t<0>(a, st);
}

}  // namespace fsvd
