// Single-query attention over a RANK-SPACE KV cache: the cache holds the pre-RoPE rank
// coefficients Pk, Pv [B,S,R] (shared by all heads); K is rebuilt per key tile inside the kernel
// as Pk_tile @ k_u[h]^T on the matrix cores, rotated at the keys' absolute positions, scored
// against the (already rebuilt and rotated) query, and V is never rebuilt per key: the softmax
// weights are applied to Pv in rank space, t = sum_n p_n Pv_n, and one product t @ v_u[h]^T per
// head finishes the job (the Acc[B,H,S,R] workspace idea of the reference's split-K design).
//
// Stage 1, grid (nsplit, Hk*groups, B), 4 waves: each wave owns 16 keys of a 64-key tile, and takes KS such
//   tiles per pass over R when the split is long, so that every k_u fragment it loads serves 16*KS keys
//   (the pass is bound by the L2 traffic of k_u, which every wave re-reads).
//   MFMA 16x16x32 bf16: A = Pk[16 keys x 32 r] and B = k_u[16 d x 32 r] are both contiguous along
//   r, so both operands are plain 16-byte global loads in the instruction's native lane layout.
//   The 8 accumulator tiles of a wave hold K[16 keys x 128 d]; d and d+64 sit in the same lane,
//   so the rotate-half RoPE is register-local; scores fold over the 16 lanes of a DPP row.
// Stage 2, grid (H, B): merge the splits in order, normalise, multiply by v_u[h].
//
// Caches shared by the heads with B * H * S of 2^17 and more (4096 keys of 32 heads: from there on it is the faster form
// at every batch size measured), when the caller has registered scratch: stage 1 is three launches.  The score kernel is stage 1 cut after the scores (it keeps neither softmax state nor rank-space sums,
// which frees the registers for four key sub-tiles per wave, and stages k_u as well as Pk with loads that write LDS
// directly); rank_decode_softmax_kernel turns the scores of a split into weights in place; rank_decode_pv_kernel
// accumulates p . Pv on the matrix cores for up to 32 heads at once, so that a Pv row is read once per head tile instead
// of once per head.  In the one-kernel form every head re-reads the Pv rows of its batch row from L2 (as much traffic
// again as k_u and Pk together) and multiplies them on the vector ALU.
// With one query head per kv head the score launch takes two heads per workgroup (rank_scores_pair_kernel), which share
// the Pk rows in LDS as well.
#include "common.hpp"
#include "kernels.hpp"

namespace fsvd {


constexpr int kRdThreads = 256;
constexpr int kRdTileKeys = 64;   // 4 waves x 16 keys
constexpr int kRdMaxChunks = 4;   // rank-space accumulator: R <= 4 * 512

template <class F>
__device__ __forceinline__ F ld_frag(const uint16_t* p) {
  return __builtin_bit_cast(F, *reinterpret_cast<const u32x4_t*>(p));
}
template <class F>
__device__ __forceinline__ F zero_frag() { return __builtin_bit_cast(F, u32x4_t{0u, 0u, 0u, 0u}); }

// dynamic LDS of the partial kernel: k_u stages [stage][128 d][64 r] bf16 (two, or three in the deep form), reused for the
// four waves' rank-space partials [4][kRdMaxChunks * 512] fp32 at the end; then the waves' Pk slots
template <int KS, bool PKL, bool DEEP, bool SC = false> struct RankDecodeLds {
  static constexpr int kStages = (DEEP || (SC && PKL)) ? 3 : 2;
  static constexpr int kKu = kStages * 128 * 64 * 2, kTb = 4 * kRdMaxChunks * 512 * 4;
  static constexpr int kMain = kKu > kTb ? kKu : kTb;
  static constexpr int kPkSlots = DEEP ? 3 : 1;
  static constexpr int kBytes = kMain + (PKL ? 4 * kPkSlots * KS * 2048 : 0);
};

// PKL: the Pk rows of a chunk (16 keys x 128 bytes per key sub-tile) are loaded as whole 128-byte pieces straight into an
// LDS slot of the wave and the fragments read from there, instead of 16 rows x 64 bytes per fragment load from global
// memory (Rk a multiple of 64; 13 % of the kernel's time at 16 x 4096 keys of rank 1664 was that access pattern)
// DEEP (short splits: one key tile or a few per workgroup, so the pass over r is a chain of chunk latencies): k_u chunks
// are loaded straight into a ring of three LDS stages as well, two chunks ahead, and the Pk pieces two chunks ahead into
// two slots per wave; the wave's load counter and one barrier per chunk are the synchronisation.  Batch 1, 512 keys,
// rank 1024: 24 us -> see the launcher.
// SC (long caches, scratch registered): the kernel stops at the scores.  It writes s[b, key, h] = q_h . K_key * scale to
// a.scores and leaves the softmax and the rank-space accumulation to rank_decode_softmax_kernel / rank_decode_pv_kernel,
// which read every Pv row once for a group of heads instead of once per head.
template <int DT, int REP, int KS, bool PKL, bool DEEP = false, bool SC = false>
__global__ __launch_bounds__(kRdThreads, 2) void rank_decode_partial_kernel(RankDecodeArgs a) {
  typedef E16<DT> E;
  typedef typename E::frag_t frag_t;
  static_assert(!DEEP || (PKL && KS == 1), "the deep form is built for single sub-tiles with Pk through LDS");
  constexpr int DH = 128, NT = DH / 16, HALF = DH / 2;
  __shared__ float wm[4][REP], wl[4][REP];
  // one LDS block, used twice: k_u chunks [2][128 d][64 r] bf16 while the keys stream, the four waves'
  // rank-space partials [4][kRdMaxChunks*512] fp32 for the merge at the end
  // 128-byte rows, 16-byte piece c of row d stored at piece c ^ (d % 8): a 16-byte LDS read is served 16 lanes a cycle
  // (lanes 0-3, 12-15, 20-27 / 4-11, 16-19, 28-31 of a half wave), and with this placement the fragment reads (lane =
  // row % 16 + 16 * piece) touch every bank once per group (rows padded to 144 bytes put two lanes on a bank)
  constexpr int KROW = 64;
  typedef RankDecodeLds<KS, PKL, DEEP, SC> Lds;
  extern __shared__ __align__(16) unsigned char rd_smem[];
  unsigned char* smem = rd_smem;                                 // k_u stages, then the waves' partials
  unsigned char* pkslot = rd_smem + Lds::kMain;                  // [wave][slot][sub-tile][16 keys][128 bytes]
  uint16_t (*kus)[DH][KROW] = reinterpret_cast<uint16_t (*)[DH][KROW]>(smem);
  float (*tbuf)[kRdMaxChunks * 512] = reinterpret_cast<float (*)[kRdMaxChunks * 512]>(smem);
  // the queries on their way to registers: in the k_u block before its first chunk takes the place; in the deep form,
  // whose first chunks are already in flight by then, in the third Pk slot of wave 0 (first written for chunk 2)
  constexpr bool kLate = DEEP && REP == 1;         // (with several heads per workgroup the registers do not reach)
  float (*qs)[DH] = reinterpret_cast<float (*)[DH]>(kLate ? pkslot + 2 * KS * 2048 : smem);

  const int groups = a.H / a.Hk / REP;             // q-head groups per kv head handled by separate blocks
  // neighbours on one XCD share an L2: the head groups of one key range (they read the same cache rows), or, when the
  // head bases outweigh the cache rows of the call (short caches, small batches), the key ranges of one head group
  const int GY = gridDim.y;
  const int t = xcd_run_index(blockIdx.x + (int)gridDim.x * (blockIdx.y + GY * blockIdx.z), (int)gridDim.x * GY * gridDim.z);
  const int gy = a.split_major ? (t / (int)gridDim.x) % GY : t % GY;
  const int s = a.split_major ? t % (int)gridDim.x : (t / GY) % (int)gridDim.x, b = t / (GY * (int)gridDim.x);
  const int hk = gy / groups, grp = gy % groups;
  const int h0 = hk * (a.H / a.Hk) + grp * REP;    // first q head of this block
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lr = lane & 15, lg = lane >> 4;        // column-in-tile / row group

  int n_keys = a.seqlens[b] + a.seqlen_add;
  n_keys = max(0, min(n_keys, a.S));
  int per = (n_keys + a.nsplit - 1) / a.nsplit;
  per = (per + kRdTileKeys - 1) / kRdTileKeys * kRdTileKeys;
  const int k0 = min(s * per, n_keys), k1 = min(n_keys, k0 + per);

  // queries of this block as fp32 through LDS into registers, rotated at position n_keys-1 when asked to
  float qv[REP][NT];
  const auto load_queries = [&]() {
    for (int i = tid; i < REP * HALF; i += kRdThreads) {
      const int g = i / HALF, d = i % HALF;
      const uint16_t* qp = a.q + (int64_t)b * a.sq_b + (int64_t)(h0 + g) * a.sq_h;
      float x0 = E::val(qp[d]), x1 = E::val(qp[d + HALF]);
      if (a.rotate_q) {
        const int tp = min(max(n_keys - 1, 0), a.rope_len - 1);
        const float c = E::val(a.cos[(int64_t)tp * HALF + d]), sn = E::val(a.sin[(int64_t)tp * HALF + d]);
        const float r0 = x0 * c - x1 * sn, r1 = x0 * sn + x1 * c;
        x0 = r0; x1 = r1;
      }
      qs[g][d] = x0 * a.scale;
      qs[g][d + HALF] = x1 * a.scale;
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < REP; ++g)
#pragma unroll
      for (int t = 0; t < NT; ++t) qv[g][t] = qs[g][(t / 4) * HALF + lr * 4 + (t % 4)];
    __syncthreads();                                               // the queries are in registers: the LDS block is free
  };
  if constexpr (!kLate) load_queries();                            // (else under the loads of the first chunk)

  const int nchunk = (a.Rv + 511) / 512;
  float m_run[REP], l_run[REP];
  float tacc[REP][kRdMaxChunks][8];
#pragma unroll
  for (int g = 0; g < REP; ++g) {
    m_run[g] = -INFINITY; l_run[g] = 0.f;
#pragma unroll
    for (int c = 0; c < kRdMaxChunks; ++c)
#pragma unroll
      for (int i = 0; i < 8; ++i) tacc[g][c][i] = 0.f;
  }

  const uint16_t* pk_b = a.pk + (int64_t)b * a.spk_b + (int64_t)hk * a.spk_h;
  const uint16_t* pv_b = a.pv + (int64_t)b * a.spv_b + (int64_t)hk * a.spv_h;
  const uint16_t* ku_h = a.k_u + (int64_t)hk * DH * a.ldku;

  for (int kt = k0; kt < k1; kt += kRdTileKeys * KS) {
    // KS key sub-tiles per pass share every k_u fragment: sub-tile j of this wave starts at kt + (4j + wave) * 16
    // ---- K tiles = Pk[16 keys, R] @ k_u[h]^T on the matrix cores.  k_u streams through LDS in 64-wide chunks of r,
    // loaded once per workgroup (thread -> row tid/2, 32 r) and double-buffered; Pk fragments come straight from
    // global memory in the instruction's lane layout.  Waves past the end of the split keep pace (clamped keys)
    // because the chunk hand-over is a block barrier.
    f32x4_t accs[KS][NT];
    const uint16_t* arow[KS];
#pragma unroll
    for (int j = 0; j < KS; ++j) {
#pragma unroll
      for (int t = 0; t < NT; ++t) accs[j][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      const int akey = min(kt + (4 * j + wave) * 16 + lr, k1 - 1);
      arow[j] = pk_b + (int64_t)akey * a.spk_s + lg * 8;
    }
    // LDS row t*16 + lr holds head dimension d = (t/4)*64 + lr*4 + t%4: a lane's accumulator tiles t = 0..3 then
    // cover four consecutive d (one 8-byte read of the rotation tables per key), tiles t and t+4 the rotate-half pair
    const int krow = tid >> 1, kcol = (tid & 1) * 32;
    const int kd = ((krow >> 4) / 4) * HALF + (krow & 15) * 4 + ((krow >> 4) % 4);
    const uint16_t* kug = ku_h + (int64_t)kd * a.ldku + kcol;
    const int nstep = (a.Rk + 63) / 64;
    u32x4_t kreg[4];
    frag_t af[KS][2];
    const auto load_ku = [&](int r0) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        kreg[i] = (r0 + kcol + i * 8 < a.Rk) ? *reinterpret_cast<const u32x4_t*>(kug + r0 + i * 8) : u32x4_t{0u, 0u, 0u, 0u};
    };
    const auto store_ku = [&](int buf) {
#pragma unroll
      for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4_t*>(&kus[buf][krow][(((kcol >> 3) + i) ^ (krow & 7)) * 8]) = kreg[i];
    };
    const auto load_pk = [&](int r0) {
#pragma unroll
      for (int j = 0; j < KS; ++j)
#pragma unroll
        for (int k = 0; k < 2; ++k) af[j][k] = (r0 + k * 32 + lg * 8 < a.Rk) ? ld_frag<frag_t>(arow[j] + r0 + k * 32) : zero_frag<frag_t>();
    };
    // PKL: lane -> key row lane / 8 (+ 8 per instruction) and the piece that belongs at LDS position lane % 8 of that row
    // (position p of row r holds piece p ^ r % 8: conflict-free 16-byte fragment reads)
    typedef const __attribute__((address_space(1))) void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    unsigned char* myslot = pkslot + (PKL ? wave * Lds::kPkSlots * KS * 2048 : 0);
    const uint16_t* prow[KS][2];
    if (PKL) {
#pragma unroll
      for (int j = 0; j < KS; ++j)
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int row = i * 8 + (lane >> 3);
          const int pkey = min(kt + (4 * j + wave) * 16 + row, k1 - 1);
          prow[j][i] = pk_b + (int64_t)pkey * a.spk_s + (((lane & 7) ^ (row & 7)) * 8);
        }
    }
    const auto issue_pk = [&](int r0) {
#pragma unroll
      for (int j = 0; j < KS; ++j)
#pragma unroll
        for (int i = 0; i < 2; ++i)
          __builtin_amdgcn_global_load_lds((gptr_t)(prow[j][i] + r0), (lptr_t)(myslot + j * 2048 + i * 1024), 16, 0, 0);
    };
    const auto read_pk = [&]() {
#pragma unroll
      for (int j = 0; j < KS; ++j)
#pragma unroll
        for (int k = 0; k < 2; ++k)
          af[j][k] = *reinterpret_cast<const frag_t*>(myslot + j * 2048 + lr * 128 + (((k * 4 + lg) ^ (lr & 7)) * 16));
    };
    // deep form, one head per workgroup: the rotation table rows of the wave's keys are requested ahead of the pass over
    // r (they are needed right behind it, and a first read from memory takes as long as several chunks)
    constexpr bool kTablesAhead = kLate;
    uint2 cwp[4], swp[4];
    if constexpr (kTablesAhead) {
      if (a.cos) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int pos = min(kt + wave * 16 + lg * 4 + i, a.rope_len - 1);
          cwp[i] = *reinterpret_cast<const uint2*>(a.cos + (int64_t)pos * HALF + lr * 4);
          swp[i] = *reinterpret_cast<const uint2*>(a.sin + (int64_t)pos * HALF + lr * 4);
        }
      }
    }
    if constexpr (DEEP) {
      // lane -> LDS row wave * 32 + i * 8 + lane / 8 and position lane % 8 of a stage; the row holds head dimension kd(row)
      // and its position p the piece p ^ row % 8 (the placement store_ku gives the register form)
      const uint16_t* kusrc[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int row = wave * 32 + i * 8 + (lane >> 3);
        const int rd = ((row >> 4) / 4) * HALF + (row & 15) * 4 + ((row >> 4) % 4);
        kusrc[i] = ku_h + (int64_t)rd * a.ldku + (((lane & 7) ^ (row & 7)) * 8);
      }
      constexpr int kGroup = 6;                    // loads per chunk and wave: four of k_u, two of Pk
      const auto issue_group = [&](int c) {
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 4; ++i)
          __builtin_amdgcn_global_load_lds((gptr_t)(kusrc[i] + c * 64), (lptr_t)(smem + (c % 3) * (DH * KROW * 2) + (wave * 32 + i * 8) * 128), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < 2; ++i)
          __builtin_amdgcn_global_load_lds((gptr_t)(prow[0][i] + c * 64), (lptr_t)(myslot + (c % 3) * 2048 + i * 1024), 16, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      };
      constexpr int kNoLgkm = (7 << 4) | (15 << 8);              // wait on the load counter only
      // (the barrier that ended the previous tile freed every stage and slot)
      issue_group(0);
      if constexpr (kLate) {
        if (kt == k0) load_queries();                            // its barriers also wait for chunk 0, which it would have anyway
      }
      if (nstep > 1) issue_group(1);
      for (int st = 0; st < nstep; ++st) {
        // chunk st has landed once only the group issued after it is outstanding
        if (st + 1 < nstep) __builtin_amdgcn_s_waitcnt(kNoLgkm | kGroup);
        else __builtin_amdgcn_s_waitcnt(kNoLgkm | 0);
        __builtin_amdgcn_sched_barrier(0);
        // the wave's own Pk fragments: slot st % 3 is next written for chunk st + 3, requested in step st + 1 behind that
        // step's reads, which these precede in the LDS queue
#pragma unroll
        for (int k = 0; k < 2; ++k)
          af[0][k] = *reinterpret_cast<const frag_t*>(myslot + (st % 3) * 2048 + lr * 128 + (((k * 4 + lg) ^ (lr & 7)) * 16));
        // everyone's pieces of chunk st are in, and stage (st - 1) % 3 is read out (its fragments fed matrix products that
        // precede this point).  The bare barrier instruction: __syncthreads() carries a fence that waits for ALL of the
        // wave's loads, the chunks requested ahead included
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const int cur = st % 3;
        // all sixteen k_u fragments of the chunk are requested before the first product: read two at a time (what the
        // compiler makes of a loop that reads and multiplies in turn), the chunk costs eight LDS round trips in a row,
        // and with one key tile per workgroup nothing else is there to hide them; the requests for chunk st + 2 go out
        // behind the reads, under their latency
        // (with several heads per workgroup the rank-space sums leave no registers for that: half a chunk at a time)
        if constexpr (REP == 1) {
          frag_t bf[2][NT];
#pragma unroll
          for (int k = 0; k < 2; ++k)
#pragma unroll
            for (int t = 0; t < NT; ++t) bf[k][t] = __builtin_bit_cast(frag_t, *reinterpret_cast<const u32x4_t*>(&kus[cur][t * 16 + lr][((k * 4 + lg) ^ (lr & 7)) * 8]));
          if (st + 2 < nstep) issue_group(st + 2);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int k = 0; k < 2; ++k)
#pragma unroll
            for (int t = 0; t < NT; ++t) accs[0][t] = E::mfma(af[0][k], bf[k][t], accs[0][t]);
        } else {
          if (st + 2 < nstep) issue_group(st + 2);
#pragma unroll
          for (int k = 0; k < 2; ++k) {
            frag_t bf[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) bf[t] = __builtin_bit_cast(frag_t, *reinterpret_cast<const u32x4_t*>(&kus[cur][t * 16 + lr][((k * 4 + lg) ^ (lr & 7)) * 8]));
#pragma unroll
            for (int t = 0; t < NT; ++t) accs[0][t] = E::mfma(af[0][k], bf[t], accs[0][t]);
          }
        }
      }
      __syncthreads();                                           // the last stages are read out before the next tile refills them
    } else if constexpr (PKL && SC) {
      // k_u chunks straight into LDS stages as well (no registers, no LDS stores): lane -> LDS row
      // wave * 32 + i * 8 + lane / 8 and position lane % 8 of the stage, which holds piece (lane % 8) ^ (row % 8) of head
      // dimension kd(row) -- the placement store_ku gives the register form.  Addresses are a wave-uniform base plus a
      // 32-bit byte offset per lane (the launcher checks that the cache of a batch row fits): no 64-bit pointer per piece
      // to keep and to advance
      uint32_t kuoff[4], pkoff[KS][2];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int row = wave * 32 + i * 8 + (lane >> 3);
        const int rd = ((row >> 4) / 4) * HALF + (row & 15) * 4 + ((row >> 4) % 4);
        kuoff[i] = (uint32_t)((rd * (int)a.ldku + (((lane & 7) ^ (row & 7)) * 8)) * 2);
      }
#pragma unroll
      for (int j = 0; j < KS; ++j)
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int row = i * 8 + (lane >> 3);
          const int pkey = min(kt + (4 * j + wave) * 16 + row, k1 - 1);
          pkoff[j][i] = (uint32_t)pkey * (uint32_t)(a.spk_s * 2) + (uint32_t)((((lane & 7) ^ (row & 7)) * 8) * 2);
        }
      const char* kub = reinterpret_cast<const char*>(ku_h);
      const char* pkb = reinterpret_cast<const char*>(pk_b);
      const auto issue_ku = [&](int c) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          __builtin_amdgcn_global_load_lds((gptr_t)(kub + c * 128 + (size_t)kuoff[i]), (lptr_t)(smem + (c % 3) * (DH * KROW * 2) + (wave * 32 + i * 8) * 128), 16, 0, 0);
      };
      const auto issue_pk = [&](int c) {
#pragma unroll
        for (int j = 0; j < KS; ++j)
#pragma unroll
          for (int i = 0; i < 2; ++i)
            __builtin_amdgcn_global_load_lds((gptr_t)(pkb + c * 128 + (size_t)pkoff[j][i]), (lptr_t)(myslot + j * 2048 + i * 1024), 16, 0, 0);
      };
      // k_u chunks run two ahead through a ring of three stages, the Pk pieces one ahead (a wave reads its slot out at the
      // top of a step and refills it at once); the wave's load counter and one barrier per step are the synchronisation.
      // Requests in issue order: ... Pk(st) [2 KS], k_u(st + 1) [4]: chunk st is complete once only the 4 newest are out.
      // (the barrier that ended the previous tile freed every stage and the slot)
      constexpr int kNoLgkm = (7 << 4) | (15 << 8);              // wait on the load counter only
      issue_ku(0);
      issue_pk(0);
      if (nstep > 1) issue_ku(1);
      for (int st = 0; st < nstep; ++st) {
        if (st + 1 < nstep) __builtin_amdgcn_s_waitcnt(kNoLgkm | 4);
        else __builtin_amdgcn_s_waitcnt(kNoLgkm | 0);
        __builtin_amdgcn_sched_barrier(0);
        read_pk();
        __builtin_amdgcn_s_waitcnt(0xc07f);         // LDS reads done (fragments in registers, the previous step's k_u reads too); loads stay in flight
        // everybody's pieces of chunk st are in, stage (st + 2) % 3 is read out (step st - 1), the slot is free.  The bare
        // barrier instruction: __syncthreads() carries a fence that waits for all of the wave's loads, the chunk requested
        // ahead included
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (st + 1 < nstep) issue_pk(st + 1);
        if (st + 2 < nstep) issue_ku(st + 2);
        __builtin_amdgcn_sched_barrier(0);
        const int cur = st % 3;
        // k_u fragments two at a time, the next two requested before the products of the current two (as in
        // rank_scores_pair_kernel: left to itself the compiler reads a pair, waits for it and multiplies)
        const auto rd_b = [&](int k, int t) {
          return __builtin_bit_cast(frag_t, *reinterpret_cast<const u32x4_t*>(&kus[cur][t * 16 + lr][((k * 4 + lg) ^ (lr & 7)) * 8]));
        };
        frag_t bq[2][2];
        bq[0][0] = rd_b(0, 0);
        bq[0][1] = rd_b(0, 1);
#pragma unroll
        for (int it = 0; it < NT; ++it) {          // item = (k, pair of tiles): k = it / 4, tiles 2 (it % 4), + 1
          const int k = it / (NT / 2), t0 = 2 * (it % (NT / 2));
          if (it + 1 < NT) {
            const int kn = (it + 1) / (NT / 2), tn = 2 * ((it + 1) % (NT / 2));
            bq[(it + 1) & 1][0] = rd_b(kn, tn);
            bq[(it + 1) & 1][1] = rd_b(kn, tn + 1);
          }
#pragma unroll
          for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int j = 0; j < KS; ++j) accs[j][t0 + tt] = E::mfma(af[j][k], bq[it & 1][tt], accs[j][t0 + tt]);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);        // the first pair (the Pk fragments are in registers)
#pragma unroll
        for (int it = 0; it + 1 < NT; ++it) {
          __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 2 * KS, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 2 * KS, 0);
      }
      __syncthreads();                             // the last stages are read out before the next tile refills them
    } else {
    // (the barrier that ended the previous tile's last chunk also freed both buffers)
    load_ku(0);
    if (PKL) issue_pk(0); else load_pk(0);
    store_ku(0);
    __syncthreads();
    for (int st = 0; st < nstep; ++st) {
      const int cur = st & 1;
      if (PKL) {
        // the chunk's pieces were requested a whole step ago: wait for them, take the fragments into registers, and
        // hand the slot to the next chunk at once
        __builtin_amdgcn_s_waitcnt(0);
        read_pk();
        __builtin_amdgcn_s_waitcnt(0);
        __builtin_amdgcn_sched_barrier(0);
        if (st + 1 < nstep) issue_pk((st + 1) * 64);
      }
      if (st + 1 < nstep) load_ku((st + 1) * 64);
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        frag_t bf[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) bf[t] = __builtin_bit_cast(frag_t, *reinterpret_cast<const u32x4_t*>(&kus[cur][t * 16 + lr][((k * 4 + lg) ^ (lr & 7)) * 8]));
#pragma unroll
        for (int j = 0; j < KS; ++j)
#pragma unroll
          for (int t = 0; t < NT; ++t) accs[j][t] = E::mfma(af[j][k], bf[t], accs[j][t]);
      }
      if (st + 1 < nstep) {
        if (!PKL) load_pk((st + 1) * 64);          // lands while the chunk is handed over
        store_ku(cur ^ 1);
      }
      __syncthreads();
    }
    }
#pragma unroll
    for (int j = 0; j < KS; ++j) {
    const int wkey0 = kt + (4 * j + wave) * 16;    // first key of this sub-tile
    if (wkey0 >= k1) break;                        // wave-uniform; later sub-tiles start even further out
    f32x4_t (&acc)[NT] = accs[j];
    // ---- rotate-half RoPE at absolute key positions (register-local: tiles t and t+4 pair up)
    if (a.cos) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int pos = min(wkey0 + lg * 4 + i, a.rope_len - 1);
        const uint2 cw = kTablesAhead ? cwp[i] : *reinterpret_cast<const uint2*>(a.cos + (int64_t)pos * HALF + lr * 4);
        const uint2 sw = kTablesAhead ? swp[i] : *reinterpret_cast<const uint2*>(a.sin + (int64_t)pos * HALF + lr * 4);
        const float cv[4] = {E::lo(cw.x), E::hi(cw.x), E::lo(cw.y), E::hi(cw.y)};
        const float sv[4] = {E::lo(sw.x), E::hi(sw.x), E::lo(sw.y), E::hi(sw.y)};
#pragma unroll
        for (int t = 0; t < NT / 2; ++t) {
          const float x0 = acc[t][i], x1 = acc[t + NT / 2][i];
          acc[t][i] = x0 * cv[t] - x1 * sv[t];
          acc[t + NT / 2][i] = x0 * sv[t] + x1 * cv[t];
        }
      }
    }
    // ---- scores, online softmax and the rank-space accumulation, per query head of the group
#pragma unroll
    for (int g = 0; g < REP; ++g) {
      float sc[4];
      float tmax = -INFINITY;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float d = 0.f;
#pragma unroll
        for (int t = 0; t < NT; ++t) d += qv[g][t] * acc[t][i];
        d = row16_sum(d);
        sc[i] = (wkey0 + lg * 4 + i < k1) ? d : -INFINITY;
        tmax = fmaxf(tmax, sc[i]);
      }
      if constexpr (SC) {
        // every lane of a row group holds the group's four scores: lane 0 of the group stores them
        if (lr == 0) {
          float* sp = a.scores + ((int64_t)b * a.H + h0 + g) * a.score_ld + wkey0 + lg * 4;
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (wkey0 + lg * 4 + i < k1) sp[i] = sc[i];
        }
        continue;
      }
      tmax = wave_max(tmax);
      const float m_new = fmaxf(m_run[g], tmax);
      const float alpha = (m_run[g] == -INFINITY) ? 0.f : __expf(m_run[g] - m_new);
      float p[4], psum = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) { p[i] = (sc[i] == -INFINITY) ? 0.f : __expf(sc[i] - m_new); psum += p[i]; }
      // every lane of a row group holds the same p; one lane per group contributes to the sum
      float pl = (lr == 0) ? psum : 0.f;
      pl = wave_sum(pl);
      l_run[g] = l_run[g] * alpha + pl;
      m_run[g] = m_new;
      // p of all 16 keys as wave-uniform values
      float pk16[16];
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) pk16[j * 4 + i] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p[i]), j * 16));
      if constexpr (REP == 1 && DEEP) {
        // one head per workgroup, one key tile: eight rows of a 512-column chunk are requested together (left to the
        // compiler, five or six rows are in flight at a time in a staggered chain of waits)
#pragma unroll
        for (int c = 0; c < kRdMaxChunks; ++c) {
          const int r = c * 512 + lane * 8;
#pragma unroll
          for (int i = 0; i < 8; ++i) tacc[g][c][i] *= alpha;
          if (c < nchunk && r < a.Rv) {
#pragma unroll
            for (int k8 = 0; k8 < 16; k8 += 8) {
              u32x4_t pvr[8];
#pragma unroll
              for (int kk = 0; kk < 8; ++kk) pvr[kk] = *reinterpret_cast<const u32x4_t*>(pv_b + (int64_t)min(wkey0 + k8 + kk, k1 - 1) * a.spv_s + r);
              __builtin_amdgcn_sched_barrier(0);
#pragma unroll
              for (int kk = 0; kk < 8; ++kk) {
                const u32x4_t v = pvr[kk];
                const float pw = pk16[k8 + kk];       // 0 for clamped keys
                tacc[g][c][0] += pw * E::lo(v.x); tacc[g][c][1] += pw * E::hi(v.x);
                tacc[g][c][2] += pw * E::lo(v.y); tacc[g][c][3] += pw * E::hi(v.y);
                tacc[g][c][4] += pw * E::lo(v.z); tacc[g][c][5] += pw * E::hi(v.z);
                tacc[g][c][6] += pw * E::lo(v.w); tacc[g][c][7] += pw * E::hi(v.w);
              }
              __builtin_amdgcn_sched_barrier(0);
            }
          }
        }
        continue;
      }
#pragma unroll
      for (int c = 0; c < kRdMaxChunks; ++c) {
        const int r = c * 512 + lane * 8;
#pragma unroll
        for (int i = 0; i < 8; ++i) tacc[g][c][i] *= alpha;
        if (c < nchunk && r < a.Rv) {
#pragma unroll
          for (int kk = 0; kk < 16; ++kk) {
            const int key = min(wkey0 + kk, k1 - 1);   // p is 0 for clamped keys
            const u32x4_t v = *reinterpret_cast<const u32x4_t*>(pv_b + (int64_t)key * a.spv_s + r);
            const float pw = pk16[kk];
            tacc[g][c][0] += pw * E::lo(v.x); tacc[g][c][1] += pw * E::hi(v.x);
            tacc[g][c][2] += pw * E::lo(v.y); tacc[g][c][3] += pw * E::hi(v.y);
            tacc[g][c][4] += pw * E::lo(v.z); tacc[g][c][5] += pw * E::hi(v.z);
            tacc[g][c][6] += pw * E::lo(v.w); tacc[g][c][7] += pw * E::hi(v.w);
          }
        }
      }
    }
    }
  }

  if constexpr (SC) return;
  // ---- merge the 4 waves (each has its own running max) and write the split's partial
#pragma unroll
  for (int g = 0; g < REP; ++g) {
    __syncthreads();
    if (lane == 0) { wm[wave][g] = m_run[g]; wl[wave][g] = l_run[g]; }
#pragma unroll
    for (int c = 0; c < kRdMaxChunks; ++c) {
#pragma unroll
      for (int i = 0; i < 8; ++i) tbuf[wave][c * 512 + lane * 8 + i] = tacc[g][c][i];
    }
    __syncthreads();
    const float M = fmaxf(fmaxf(wm[0][g], wm[1][g]), fmaxf(wm[2][g], wm[3][g]));
    float w[4], L = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) { w[j] = (wm[j][g] == -INFINITY) ? 0.f : __expf(wm[j][g] - M); L += w[j] * wl[j][g]; }
    const int64_t slot = ((int64_t)b * a.H + h0 + g) * a.nsplit + s;
    for (int r = tid; r < a.Rv; r += kRdThreads)
      a.ws_acc[slot * a.Rv + r] = w[0] * tbuf[0][r] + w[1] * tbuf[1][r] + w[2] * tbuf[2][r] + w[3] * tbuf[3][r];
    if (tid == 0) { a.ws_m[slot] = M; a.ws_l[slot] = L; }
  }
}

// The score launch for caches shared by the heads, one query head per kv head, ranks on the 64 grid: a workgroup of eight
// waves takes TWO heads over the same 64 KS keys, waves 0-3 head 2 gy and waves 4-7 head 2 gy + 1.  Wave w and wave w + 4
// work on the same key sub-tiles and read their Pk fragments from one LDS slot, which the two of them fill (half of the
// sub-tiles each): the Pk rows of a batch row cross from L2 to LDS once per pair of heads instead of once per head (at
// batch 16 x 4096 keys x rank 1664 the score launch moves 7 GB per layer through the compute units' load path instead of
// 10.5).  Every head has its own two stages of k_u chunks; both operands are requested one chunk ahead, straight into
// LDS; per chunk: the wave's load counter, one barrier (everybody's pieces of this chunk are in, everybody has left the
// previous chunk), the requests for the next chunk, the fragments, the products.  grid (nsplit, Hk / 2, B), 512 threads,
// one workgroup per compute unit (128 KB of LDS).
constexpr int kRdPairThreads = 512;
template <int KS> struct RankPairLds {
  static constexpr int kKu = 2 * 128 * 64 * 2;                   // two stages of one head's k_u chunk [128 d][64 r] bf16
  static constexpr int kSlot = KS * 2048;                        // Pk of KS sub-tiles x 16 keys x 128 bytes
  static constexpr int kBytes = 2 * kKu + 4 * 2 * kSlot;         // both heads' stages, then [pair of waves][2 slots]
};
template <int DT, int KS>
__global__ __launch_bounds__(kRdPairThreads, 1) void rank_scores_pair_kernel(RankDecodeArgs a) {
  typedef E16<DT> E;
  typedef typename E::frag_t frag_t;
  static_assert(KS == 2 || KS == 4, "the two waves of a pair fill half of the sub-tiles each");
  constexpr int DH = 128, NT = DH / 16, HALF = DH / 2, KROW = 64;
  typedef RankPairLds<KS> Lds;
  typedef const __attribute__((address_space(1))) void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;
  extern __shared__ __align__(16) unsigned char rd_smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hp = wave >> 2, w4 = wave & 3;
  const int lr = lane & 15, lg = lane >> 4;
  unsigned char* kubase = rd_smem + hp * Lds::kKu;                // this head's two k_u stages
  unsigned char* slots = rd_smem + 2 * Lds::kKu + w4 * 2 * Lds::kSlot;   // the pair's two Pk slots
  uint16_t (*kus)[DH][KROW] = reinterpret_cast<uint16_t (*)[DH][KROW]>(kubase);
  float (*qs)[DH] = reinterpret_cast<float (*)[DH]>(rd_smem);      // the two queries, before the first chunk takes the place

  const int GY = gridDim.y;
  const int t = xcd_run_index(blockIdx.x + (int)gridDim.x * (blockIdx.y + GY * blockIdx.z), (int)gridDim.x * GY * gridDim.z);
  const int gy = t % GY, s = (t / GY) % (int)gridDim.x, b = t / (GY * (int)gridDim.x);
  const int h = 2 * gy + hp;                       // query head = kv head

  int n_keys = a.seqlens[b] + a.seqlen_add;
  n_keys = max(0, min(n_keys, a.S));
  int per = (n_keys + a.nsplit - 1) / a.nsplit;
  per = (per + kRdTileKeys - 1) / kRdTileKeys * kRdTileKeys;
  const int k0 = min(s * per, n_keys), k1 = min(n_keys, k0 + per);

  for (int i = tid; i < 2 * HALF; i += kRdPairThreads) {
    const int g = i / HALF, d = i % HALF;
    const uint16_t* qp = a.q + (int64_t)b * a.sq_b + (int64_t)(2 * gy + g) * a.sq_h;
    float x0 = E::val(qp[d]), x1 = E::val(qp[d + HALF]);
    if (a.rotate_q) {
      const int tp = min(max(n_keys - 1, 0), a.rope_len - 1);
      const float c = E::val(a.cos[(int64_t)tp * HALF + d]), sn = E::val(a.sin[(int64_t)tp * HALF + d]);
      const float r0 = x0 * c - x1 * sn, r1 = x0 * sn + x1 * c;
      x0 = r0; x1 = r1;
    }
    qs[g][d] = x0 * a.scale;
    qs[g][d + HALF] = x1 * a.scale;
  }
  __syncthreads();
  float qv[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) qv[t] = qs[hp][(t / 4) * HALF + lr * 4 + (t % 4)];
  __syncthreads();                                                 // the queries are in registers: the LDS block is free

  const char* pkb = reinterpret_cast<const char*>(a.pk + (int64_t)b * a.spk_b);
  const char* kub = reinterpret_cast<const char*>(a.k_u + (int64_t)h * DH * a.ldku);
  const int nstep = a.Rk / 64;
  // k_u: lane -> LDS row w4 * 32 + i * 8 + lane / 8 and position lane % 8 of a stage, which holds piece (lane % 8) ^ (row % 8)
  // of head dimension kd(row): row t * 16 + lr of a stage is head dimension (t / 4) * 64 + lr * 4 + t % 4, so that a
  // lane's accumulator tiles t = 0..3 cover four consecutive dimensions and tiles t, t + 4 a rotation pair
  uint32_t kuoff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = w4 * 32 + i * 8 + (lane >> 3);
    const int rd = ((row >> 4) / 4) * HALF + (row & 15) * 4 + ((row >> 4) % 4);
    kuoff[i] = (uint32_t)((rd * (int)a.ldku + (((lane & 7) ^ (row & 7)) * 8)) * 2);
  }
  const auto issue_ku = [&](int c) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      __builtin_amdgcn_global_load_lds((gptr_t)(kub + c * 128 + (size_t)kuoff[i]), (lptr_t)(kubase + (c & 1) * (DH * KROW * 2) + (w4 * 32 + i * 8) * 128), 16, 0, 0);
  };

  for (int kt = k0; kt < k1; kt += kRdTileKeys * KS) {
    // sub-tile j of the pair starts at key kt + (4 j + w4) * 16; this wave requests sub-tiles hp * KS / 2 .. + KS / 2
    f32x4_t accs[KS][NT];
#pragma unroll
    for (int j = 0; j < KS; ++j)
#pragma unroll
      for (int t = 0; t < NT; ++t) accs[j][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    uint32_t pkoff[KS / 2][2];
#pragma unroll
    for (int jj = 0; jj < KS / 2; ++jj)
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int j = hp * (KS / 2) + jj, row = i * 8 + (lane >> 3);
        const int pkey = min(kt + (4 * j + w4) * 16 + row, k1 - 1);
        pkoff[jj][i] = (uint32_t)pkey * (uint32_t)(a.spk_s * 2) + (uint32_t)((((lane & 7) ^ (row & 7)) * 8) * 2);
      }
    const auto issue_pk = [&](int c) {
#pragma unroll
      for (int jj = 0; jj < KS / 2; ++jj)
#pragma unroll
        for (int i = 0; i < 2; ++i)
          __builtin_amdgcn_global_load_lds((gptr_t)(pkb + c * 128 + (size_t)pkoff[jj][i]),
                                           (lptr_t)(slots + (c & 1) * Lds::kSlot + (hp * (KS / 2) + jj) * 2048 + i * 1024), 16, 0, 0);
    };
    // (the barrier that ended the previous tile freed every stage and slot)
    issue_ku(0);
    issue_pk(0);
    for (int st = 0; st < nstep; ++st) {
      __builtin_amdgcn_s_waitcnt(0);               // this wave's pieces of chunk st have landed (and its LDS reads of chunk st - 1 are done)
      // everybody's pieces of chunk st are in; everybody has left chunk st - 1, whose stage and slot take chunk st + 1.  The
      // bare barrier instruction (nothing is in flight here that a fence would have to wait for)
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      if (st + 1 < nstep) { issue_pk(st + 1); issue_ku(st + 1); }
      __builtin_amdgcn_sched_barrier(0);
      const int cur = st & 1;
      const unsigned char* slot = slots + cur * Lds::kSlot;
      frag_t af[KS][2];
#pragma unroll
      for (int j = 0; j < KS; ++j)
#pragma unroll
        for (int k = 0; k < 2; ++k)
          af[j][k] = *reinterpret_cast<const frag_t*>(slot + j * 2048 + lr * 128 + (((k * 4 + lg) ^ (lr & 7)) * 16));
      // k_u fragments two at a time, the next two requested before the products of the current two: left to itself the
      // compiler reads a pair, waits for it and multiplies, and every pair pays an LDS round trip about as long as its
      // 2 KS products (the launch then sits at half of the matrix cores' time by counter)
      const auto rd_b = [&](int k, int t) {
        return __builtin_bit_cast(frag_t, *reinterpret_cast<const u32x4_t*>(&kus[cur][t * 16 + lr][((k * 4 + lg) ^ (lr & 7)) * 8]));
      };
      frag_t bq[2][2];
      bq[0][0] = rd_b(0, 0);
      bq[0][1] = rd_b(0, 1);
#pragma unroll
      for (int it = 0; it < NT; ++it) {            // item = (k, pair of tiles): k = it / 4, tiles 2 (it % 4), + 1
        const int k = it / (NT / 2), t0 = 2 * (it % (NT / 2));
        if (it + 1 < NT) {
          const int kn = (it + 1) / (NT / 2), tn = 2 * ((it + 1) % (NT / 2));
          bq[(it + 1) & 1][0] = rd_b(kn, tn);
          bq[(it + 1) & 1][1] = rd_b(kn, tn + 1);
        }
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
          for (int j = 0; j < KS; ++j) accs[j][t0 + tt] = E::mfma(af[j][k], bq[it & 1][tt], accs[j][t0 + tt]);
      }
      // the order asked of the scheduler: the Pk fragments and the first pair; then, seven times, the next pair's two
      // reads in front of the current pair's 2 KS products; then the last pair's products
      __builtin_amdgcn_sched_group_barrier(0x100, 2 * KS + 2, 0);
#pragma unroll
      for (int it = 0; it + 1 < NT; ++it) {
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 2 * KS, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 2 * KS, 0);
    }
    __syncthreads();                               // the last chunk is read out before the next tile refills the stages
#pragma unroll
    for (int j = 0; j < KS; ++j) {
      const int wkey0 = kt + (4 * j + w4) * 16;    // first key of this sub-tile
      if (wkey0 >= k1) break;                      // wave-uniform; later sub-tiles start even further out
      f32x4_t (&acc)[NT] = accs[j];
      if (a.cos) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int pos = min(wkey0 + lg * 4 + i, a.rope_len - 1);
          const uint2 cw = *reinterpret_cast<const uint2*>(a.cos + (int64_t)pos * HALF + lr * 4);
          const uint2 sw = *reinterpret_cast<const uint2*>(a.sin + (int64_t)pos * HALF + lr * 4);
          const float cv[4] = {E::lo(cw.x), E::hi(cw.x), E::lo(cw.y), E::hi(cw.y)};
          const float sv[4] = {E::lo(sw.x), E::hi(sw.x), E::lo(sw.y), E::hi(sw.y)};
#pragma unroll
          for (int t = 0; t < NT / 2; ++t) {
            const float x0 = acc[t][i], x1 = acc[t + NT / 2][i];
            acc[t][i] = x0 * cv[t] - x1 * sv[t];
            acc[t + NT / 2][i] = x0 * sv[t] + x1 * cv[t];
          }
        }
      }
      float sc[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float d = 0.f;
#pragma unroll
        for (int t = 0; t < NT; ++t) d += qv[t] * acc[t][i];
        sc[i] = row16_sum(d);
      }
      if (lr == 0) {
        float* sp = a.scores + ((int64_t)b * a.H + h) * a.score_ld + wkey0 + lg * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (wkey0 + lg * 4 + i < k1) sp[i] = sc[i];
      }
    }
  }
}

// Softmax weights of one split of one (batch row, head), in place: the scores s[b, h, key] of the split become the
// weights p = exp(s - m[b,h,split]) in the form the accumulation kernel multiplies with, and the split's maximum and sum
// go to ws_m / ws_l (the merge kernel folds the splits as it does for the one-kernel form).  Every group of 8 keys (32
// bytes of the row) is rewritten as two matrix-core fragments of 8 bf16 each: hi = bf16(p) of the 8 keys, then
// lo = bf16(p - hi), so that hi + lo carries p to 2^-17 and the consumer needs no arithmetic on them.  Keys between the end
// of the cache row and the next multiple of 64 get weight 0.  grid (nsplit, H, B), 256 threads; rows of the score buffer
// are a.score_ld floats apart (a multiple of 64).
template <int DT>
__global__ __launch_bounds__(kRdThreads) void rank_decode_softmax_kernel(RankDecodeArgs a) {
  typedef E16<DT> E;
  typedef typename E::frag_t frag_t;
  __shared__ float red[4];
  const int s = blockIdx.x, h = blockIdx.y, b = blockIdx.z, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int n_keys = a.seqlens[b] + a.seqlen_add;
  n_keys = max(0, min(n_keys, a.S));
  int per = (n_keys + a.nsplit - 1) / a.nsplit;
  per = (per + kRdTileKeys - 1) / kRdTileKeys * kRdTileKeys;
  const int k0 = min(s * per, n_keys), k1 = min(n_keys, k0 + per);
  if (k0 >= k1) {
    if (tid == 0) {
      const int64_t slot = ((int64_t)b * a.H + h) * a.nsplit + s;
      a.ws_m[slot] = -INFINITY;                    // an empty split: the merge gives it weight 0
      a.ws_l[slot] = 0.f;
    }
    return;
  }
  float* sp = a.scores + ((int64_t)b * a.H + h) * a.score_ld;
  const int kend = (k1 + 63) / 64 * 64;            // k0 is a multiple of 64; only the last split of a row ends off the grid
  // a thread takes groups of 8 keys: both passes read the same 32 bytes, the second rewrites them
  float m = -INFINITY;
  for (int k = k0 + tid * 8; k < k1; k += kRdThreads * 8) {
    const f32x4_t x0 = *reinterpret_cast<const f32x4_t*>(sp + k), x1 = *reinterpret_cast<const f32x4_t*>(sp + k + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (k + i < k1) m = fmaxf(m, x0[i]);
      if (k + 4 + i < k1) m = fmaxf(m, x1[i]);
    }
  }
  m = wave_max(m);
  if (lane == 0) red[wave] = m;
  __syncthreads();
  const float M = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  float l = 0.f;
  for (int k = k0 + tid * 8; k < kend; k += kRdThreads * 8) {
    const f32x4_t x0 = *reinterpret_cast<const f32x4_t*>(sp + k), x1 = *reinterpret_cast<const f32x4_t*>(sp + k + 4);
    uint32_t hi[8], lo[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float p = (k + i < k1) ? __expf((i < 4 ? x0[i] : x1[i - 4]) - M) : 0.f;
      l += p;
      hi[i] = E::bits(p);
      lo[i] = E::bits(p - E::val(hi[i]));
    }
    uint32_t* wp = reinterpret_cast<uint32_t*>(sp + k);
    *reinterpret_cast<u32x4_t*>(wp) = u32x4_t{hi[0] | (hi[1] << 16), hi[2] | (hi[3] << 16), hi[4] | (hi[5] << 16), hi[6] | (hi[7] << 16)};
    *reinterpret_cast<u32x4_t*>(wp + 4) = u32x4_t{lo[0] | (lo[1] << 16), lo[2] | (lo[3] << 16), lo[4] | (lo[5] << 16), lo[6] | (lo[7] << 16)};
  }
  l = wave_sum(l);
  if (lane == 0) red[wave] = l;
  __syncthreads();
  if (tid == 0) {
    const int64_t slot = ((int64_t)b * a.H + h) * a.nsplit + s;
    a.ws_m[slot] = M;
    a.ws_l[slot] = ((red[0] + red[1]) + red[2]) + red[3];
  }
}

// Acc[b, h, split, r] = sum over the split's keys of p[b, h, key] * Pv[b, key, r] on the matrix cores, for 16 * MT heads at
// once: a Pv row is read once per head tile instead of once per head (coefficient caches shared by the heads only).
// grid (r slices of 128, nsplit * head tiles, B), 4 waves; wave w owns the 32 columns c0 + 32 w of the slice.  Per block of
// 64 keys the workgroup stages Pv[64 keys x 128 r] and the weight fragments of its heads (the hi and lo term the softmax
// kernel left in the score buffer, 32 bytes per head and 8 keys) in LDS, two blocks ahead in registers; a lane gathers its
// B fragment (8 keys of one column) with 2-byte LDS reads and takes its A fragments with 16-byte ones; two matrix
// products per tile so that the sum keeps fp32 weights; fp32 accumulation in key order.
template <int DT, int MT>
__global__ __launch_bounds__(kRdThreads) void rank_decode_pv_kernel(RankDecodeArgs a) {
  typedef E16<DT> E;
  typedef typename E::frag_t frag_t;
  // LDS rows: 128 columns of a key in 260 bytes (8 rows apart = 8 banks apart: the four key groups of a fragment gather
  // from disjoint banks), the 64 keys of a head in 272 bytes (16 heads read 16 bytes each from disjoint banks)
  constexpr int KB = 64, NT = 2, PITCH = 260, WPITCH = 272, HT = 16 * MT;
  __shared__ __align__(16) unsigned char tile[2][KB * PITCH];
  __shared__ __align__(16) unsigned char wtile[2][HT * WPITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lr = lane & 15, lg = lane >> 4;
  const int ntile = (a.H + HT - 1) / HT;
  const int s = blockIdx.y / ntile, ht = blockIdx.y % ntile, b = blockIdx.z;
  const int h0 = ht * HT;
  int n_keys = a.seqlens[b] + a.seqlen_add;
  n_keys = max(0, min(n_keys, a.S));
  int per = (n_keys + a.nsplit - 1) / a.nsplit;
  per = (per + kRdTileKeys - 1) / kRdTileKeys * kRdTileKeys;
  const int k0 = min(s * per, n_keys), k1 = min(n_keys, k0 + per);
  const int c0 = blockIdx.x * 128;                 // first column of the slice
  // staging of Pv: thread -> key row tid / 16 (+ 16 i) of the block, 16-byte piece tid % 16 of the 256-byte row slice
  const int srow = tid >> 4, spiece = tid & 15;
  const bool scol = c0 + spiece * 8 < a.Rv;        // Rv is a multiple of 8: a piece is inside or outside as a whole
  const uint16_t* pv_b = a.pv + (int64_t)b * a.spv_b + (scol ? c0 + spiece * 8 : 0);
  // staging of the weights: thread -> head tid / 8 of the tile (32 heads: all threads; 16 heads: the first half), the 32
  // bytes of key group tid % 8
  const int whead = tid >> 3, wgrp = tid & 7;
  const bool wlive = whead < HT && h0 + whead < a.H;
  const float* wsrc = a.scores + ((int64_t)b * a.H + (wlive ? h0 + whead : 0)) * a.score_ld + wgrp * 8;
  struct Regs { u32x4_t v[4]; u32x4_t w[2]; };
  const auto load_block = [&](int kb, Regs& r) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key = min(kb + i * 16 + srow, k1 - 1);   // clamped rows carry weight 0
      r.v[i] = scol ? __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(pv_b + (int64_t)key * a.spv_s)) : u32x4_t{0u, 0u, 0u, 0u};
    }
    const u32x4_t* p = reinterpret_cast<const u32x4_t*>(wsrc + kb);
    r.w[0] = wlive ? p[0] : u32x4_t{0u, 0u, 0u, 0u};
    r.w[1] = wlive ? p[1] : u32x4_t{0u, 0u, 0u, 0u};
  };
  const auto store_block = [&](int buf, const Regs& r) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint32_t* d = reinterpret_cast<uint32_t*>(&tile[buf][(i * 16 + srow) * PITCH + spiece * 16]);
      d[0] = r.v[i].x; d[1] = r.v[i].y; d[2] = r.v[i].z; d[3] = r.v[i].w;
    }
    if (whead < HT) {
      u32x4_t* d = reinterpret_cast<u32x4_t*>(&wtile[buf][whead * WPITCH + wgrp * 32]);
      d[0] = r.w[0];
      d[1] = r.w[1];
    }
  };
  f32x4_t acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const auto products = [&](int buf) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      u32x4_t af[MT][2];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const u32x4_t* p = reinterpret_cast<const u32x4_t*>(&wtile[buf][(mt * 16 + lr) * WPITCH + (ks * 4 + lg) * 32]);
        af[mt][0] = p[0];
        af[mt][1] = p[1];
      }
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        uint16_t e[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) e[j] = *reinterpret_cast<const uint16_t*>(&tile[buf][(ks * 32 + lg * 8 + j) * PITCH + (wave * 32 + nt * 16 + lr) * 2]);
        const u32x4_t bw{(uint32_t)e[0] | ((uint32_t)e[1] << 16), (uint32_t)e[2] | ((uint32_t)e[3] << 16),
                         (uint32_t)e[4] | ((uint32_t)e[5] << 16), (uint32_t)e[6] | ((uint32_t)e[7] << 16)};
        const frag_t bf = __builtin_bit_cast(frag_t, bw);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          acc[mt][nt] = E::mfma(__builtin_bit_cast(frag_t, af[mt][0]), bf, acc[mt][nt]);
          acc[mt][nt] = E::mfma(__builtin_bit_cast(frag_t, af[mt][1]), bf, acc[mt][nt]);
        }
      }
    }
  };
  if (k0 < k1) {
    // two register sets, each with the Pv pieces and the weights of one block: while block i is multiplied out of LDS,
    // block i + 1 sits in one set (requested an iteration ago, stored to the other tile after the products) and block i + 2
    // is requested into the other, so that two blocks per workgroup are always on their way from memory
    Regs ra, rb;
    load_block(k0, ra);
    if (k0 + KB < k1) load_block(k0 + KB, rb);
    store_block(0, ra);
    for (int kb = k0; kb < k1; kb += 2 * KB) {
      if (kb + 2 * KB < k1) load_block(kb + 2 * KB, ra);
      __syncthreads();                             // block kb is in tile 0; everybody has left tile 1
      products(0);
      if (kb + KB >= k1) break;
      store_block(1, rb);
      if (kb + 3 * KB < k1) load_block(kb + 3 * KB, rb);
      __syncthreads();                             // block kb + KB is in tile 1; everybody has left tile 0
      products(1);
      if (kb + 2 * KB >= k1) break;
      store_block(0, ra);
    }
  }
  // element i of a lane: head h0 + mt * 16 + lg * 4 + i, column c0 + wave * 32 + nt * 16 + lr
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int r = c0 + wave * 32 + nt * 16 + lr;
    if (r < a.Rv) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int h = h0 + mt * 16 + lg * 4 + i;
          if (h < a.H) a.ws_acc[(((int64_t)b * a.H + h) * a.nsplit + s) * a.Rv + r] = acc[mt][nt][i];
        }
    }
  }
}

// out[b,h,:] = (sum_s w_s Acc_s / max(sum_s w_s L_s, 1e-20)) @ v_u[h]^T (+ bv[h])
// grid (H, B, head-dimension slices): every slice merges the splits for itself (a few KB from L2) and multiplies by its
// 128 / gridDim.z rows of v_u[h]; a wave takes four rows at a time with all of their loads in flight.  With one workgroup
// per head and one row per wave at a time, a batch-1 call spent 36 us here on 32 compute units (8 MB of v_u, one load
// latency per row).
template <int DT>
__global__ __launch_bounds__(kRdThreads) void rank_decode_merge_kernel(RankDecodeArgs a) {
  typedef E16<DT> E;
  typedef typename E::frag_t frag_t;
  constexpr int DH = 128, RW = 4, NIT = kRdMaxChunks;
  __shared__ __align__(16) float ts[kRdMaxChunks * 512];
  const int h = blockIdx.x, b = blockIdx.y;
  const int rows = DH / (int)gridDim.z, d0 = (int)blockIdx.z * rows;   // gridDim.z divides 128 / (4 waves * RW) = 8
  const int hk = h / (a.H / a.Hk);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // the v_u rows of the first round are requested before the merge, which is a chain of dependent loads of its own
  u32x4_t v[RW][NIT];
  const auto load_rows = [&](int dd) {
    const uint16_t* row = a.v_u + (int64_t)(hk * DH + d0 + dd) * a.ldvu + lane * 8;
#pragma unroll
    for (int it = 0; it < NIT; ++it)
#pragma unroll
      for (int j = 0; j < RW; ++j)
        v[j][it] = (lane * 8 + it * 512 < a.Rv) ? *reinterpret_cast<const u32x4_t*>(row + (int64_t)j * a.ldvu + it * 512) : u32x4_t{0u, 0u, 0u, 0u};
  };
  load_rows(wave * RW);
  const int64_t slot0 = ((int64_t)b * a.H + h) * a.nsplit;
  // running maxima and sums of the splits: lane i of every wave takes split i (one round trip for up to 64 splits)
  float M = -INFINITY, den = 0.f;
  for (int s0 = 0; s0 < a.nsplit; s0 += 64) {
    const int sidx = s0 + lane;
    const float m = sidx < a.nsplit ? a.ws_m[slot0 + sidx] : -INFINITY;
    const float l = sidx < a.nsplit ? a.ws_l[slot0 + sidx] : 0.f;
    const float Mn = fmaxf(M, wave_max(m));
    const float part = wave_sum((m == -INFINITY) ? 0.f : __expf(m - Mn) * l);
    den = ((M == -INFINITY) ? 0.f : den * __expf(M - Mn)) + part;
    M = Mn;
  }
  const float inv = 1.0f / fmaxf(den, 1e-20f);
  // four consecutive r per thread, the loads of up to eight splits in flight at once (one split per round trip made this
  // loop the longest part of the kernel); the splits are added in order
  constexpr int SU = 8;
  for (int r = tid * 4; r < kRdMaxChunks * 512; r += kRdThreads * 4) {
    f32x4_t t = f32x4_t{0.f, 0.f, 0.f, 0.f};
    if (r < a.Rv)                                  // Rv is a multiple of 8: the four are all inside or all outside
      for (int s0 = 0; s0 < a.nsplit; s0 += SU) {
        f32x4_t x[SU];
        float w[SU];
#pragma unroll
        for (int u = 0; u < SU; ++u) {
          const int sidx = min(s0 + u, a.nsplit - 1);
          x[u] = *reinterpret_cast<const f32x4_t*>(a.ws_acc + (slot0 + sidx) * a.Rv + r);
          const float m = a.ws_m[slot0 + sidx];
          w[u] = (s0 + u < a.nsplit && m != -INFINITY) ? __expf(m - M) : 0.f;
        }
#pragma unroll
        for (int u = 0; u < SU; ++u) t += w[u] * x[u];
      }
    *reinterpret_cast<f32x4_t*>(&ts[r]) = t * inv;  // zero past Rv: the products below run over whole chunks
  }
  __syncthreads();
  uint16_t* outp = a.out + (int64_t)b * a.so_b + (int64_t)h * a.so_h;
  // wave w takes rows d0 + w * RW + j (+ 4 * RW per round); rows is a multiple of 4 * RW
  for (int dd = wave * RW; dd < rows; dd += (kRdThreads / 64) * RW) {
    if (dd != wave * RW) load_rows(dd);
    float acc[RW];
#pragma unroll
    for (int j = 0; j < RW; ++j) acc[j] = 0.f;
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int r = lane * 8 + it * 512;
      const f32x4_t t0 = *reinterpret_cast<const f32x4_t*>(&ts[r]), t1 = *reinterpret_cast<const f32x4_t*>(&ts[r + 4]);
#pragma unroll
      for (int j = 0; j < RW; ++j)
        acc[j] += t0[0] * E::lo(v[j][it].x) + t0[1] * E::hi(v[j][it].x) + t0[2] * E::lo(v[j][it].y) + t0[3] * E::hi(v[j][it].y) +
                  t1[0] * E::lo(v[j][it].z) + t1[1] * E::hi(v[j][it].z) + t1[2] * E::lo(v[j][it].w) + t1[3] * E::hi(v[j][it].w);
    }
#pragma unroll
    for (int j = 0; j < RW; ++j) {
      float o = wave_sum(acc[j]);
      if (lane == 0) {
        const int d = d0 + dd + j;
        if (a.bv) o += E::val(a.bv[hk * DH + d]);
        outp[d] = (uint16_t)E::bits(o);
      }
    }
  }
}

// floats of the score buffer with which a call of this shape runs as three launches; 0: the shape keeps the one-kernel form
size_t rank_decode_scores_floats(int B, int H, int S, int64_t spv_h) {
  if (B <= 0 || H <= 0 || S < 256 || spv_h != 0) return 0;
  const size_t n = (size_t)B * H * (((size_t)S + 63) / 64 * 64);
  return n >= ((size_t)1 << 17) ? n : 0;
}

template <int DT>
static int launch_rank_decode_t(const RankDecodeArgs& a, hipStream_t st) {
  const char* fn = "fsvd_attn_decode_rankkv";
  if (a.B <= 0 || a.H <= 0 || a.Hk <= 0 || a.H % a.Hk != 0 || a.S <= 0 || a.nsplit <= 0) {
    set_last_error("%s: bad shape B=%d H=%d Hk=%d S=%d nsplit=%d", fn, a.B, a.H, a.Hk, a.S, a.nsplit);
    return kErrBadShape;
  }
  if (a.Dh != 128) { set_last_error("%s: head_dim %d is not 128", fn, a.Dh); return kErrBadShape; }
  if (a.Rk <= 0 || a.Rv <= 0 || (a.Rk % 8) || (a.Rv % 8) || a.Rv > kRdMaxChunks * 512) {
    set_last_error("%s: ranks must be multiples of 8 with Rv <= %d (got Rk=%d Rv=%d); pad the factors", fn, kRdMaxChunks * 512, a.Rk, a.Rv);
    return kErrBadShape;
  }
  const auto mis = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) != 0; };
  if (mis(a.ws_acc)) { set_last_error("%s: the Acc workspace must be 16-byte aligned", fn); return kErrBadAlign; }
  if (mis(a.pk) || mis(a.pv) || mis(a.k_u) || mis(a.v_u) || (a.spk_s % 8) || (a.spv_s % 8) || (a.spk_b % 8) || (a.spv_b % 8) || (a.spk_h % 8) || (a.spv_h % 8) ||
      (a.ldku % 8) || (a.ldvu % 8)) {
    set_last_error("%s: cache / factor pointers and strides must be 16-byte aligned", fn);
    return kErrBadAlign;
  }
  if (a.cos && (((reinterpret_cast<uintptr_t>(a.cos) | reinterpret_cast<uintptr_t>(a.sin)) & 7) != 0)) {
    set_last_error("%s: rotation tables must be 8-byte aligned", fn);
    return kErrBadAlign;
  }
  const int rep = a.H / a.Hk;
  dim3 block(kRdThreads);
  // caches shared by the heads from 2^17 (head, key) pairs on, when the caller brings a buffer for the scores of the call
  // ([B,H,score_ld] fp32): scores -> softmax -> rank-space accumulation per head tile, as three launches.  The form
  // depends on the shape and on that argument alone, never on process state.
  const int64_t score_ld = ((int64_t)a.S + 63) / 64 * 64;
  const bool three = a.scores != nullptr && rank_decode_scores_floats(a.B, a.H, a.S, a.spv_h) != 0;
  // the one-kernel form: which operand the neighbours on an XCD share.  Every workgroup of a head group reads that
  // group's 128 x Rk rows of k_u, every workgroup of a key range the range's Pk rows: the larger set decides
  RankDecodeArgs a1 = a;
  a1.split_major = (int64_t)a.Hk * a.Dh > (int64_t)a.B * a.S && a.spk_h == 0 ? 1 : 0;
  RankDecodeArgs a3 = a;
  a3.scores = three ? a.scores : nullptr;
  a3.score_ld = score_ld;
  // key sub-tiles per pass: long splits amortise every k_u fragment over more keys (any value is correct for any
  // length; short splits would only rebuild clamped keys)
  const int per = (a.S + a.nsplit - 1) / a.nsplit;
  const int ks = per >= 128 ? 2 : 1;
  const bool pkl = (a.Rk % 64) == 0;               // whole 128-byte pieces of every Pk row
  // short splits (one sub-tile per wave and pass): the deep form, whose pass over r is not a chain of load latencies
  // (batch 1, 512 keys, rank 1024, 32 heads: 24 us per launch with chunks requested one step ahead through registers)
  const bool deep = pkl && ks == 1;
#define FSVD_RD_LAUNCH_T(REP_, KS_, PKL_, DEEP_, GY_)                                                                               \
  do {                                                                                                                              \
    constexpr int lds = RankDecodeLds<KS_, PKL_, DEEP_>::kBytes;                                                                    \
    static bool granted = false;                                                                                                    \
    if (!granted && lds >= 48 * 1024) {                                                                                             \
      hipError_t ea = hipFuncSetAttribute(reinterpret_cast<const void*>(&rank_decode_partial_kernel<DT, REP_, KS_, PKL_, DEEP_>),       \
                                          hipFuncAttributeMaxDynamicSharedMemorySize, lds);                                         \
      if (ea != hipSuccess) { set_last_error("%s: cannot reserve %d bytes of LDS: %s", fn, lds, hipGetErrorString(ea)); return kErrLaunch; } \
      granted = true;                                                                                                               \
    }                                                                                                                               \
    hipLaunchKernelGGL((rank_decode_partial_kernel<DT, REP_, KS_, PKL_, DEEP_>), dim3(a.nsplit, GY_, a.B), block, lds, st, a1);         \
  } while (0)
#define FSVD_RD_LAUNCH_SC(REP_, KS_, PKL_, GY_)                                                                                      \
  do {                                                                                                                              \
    constexpr int lds = RankDecodeLds<KS_, PKL_, false, true>::kBytes;                                                              \
    static bool granted = false;                                                                                                    \
    if (!granted && lds >= 48 * 1024) {                                                                                             \
      hipError_t ea = hipFuncSetAttribute(reinterpret_cast<const void*>(&rank_decode_partial_kernel<DT, REP_, KS_, PKL_, false, true>), \
                                          hipFuncAttributeMaxDynamicSharedMemorySize, lds);                                         \
      if (ea != hipSuccess) { set_last_error("%s: cannot reserve %d bytes of LDS: %s", fn, lds, hipGetErrorString(ea)); return kErrLaunch; } \
      granted = true;                                                                                                               \
    }                                                                                                                               \
    hipLaunchKernelGGL((rank_decode_partial_kernel<DT, REP_, KS_, PKL_, false, true>), dim3(a.nsplit, GY_, a.B), block, lds, st, a3);   \
  } while (0)
#define FSVD_RD_LAUNCH(REP_, KS_, GY_)                                                                                              \
  do {                                                                                                                              \
    if (KS_ == 1 && deep) FSVD_RD_LAUNCH_T(REP_, 1, true, true, GY_);                                                               \
    else if (pkl) FSVD_RD_LAUNCH_T(REP_, KS_, true, false, GY_);                                                                    \
    else FSVD_RD_LAUNCH_T(REP_, KS_, false, false, GY_);                                                                            \
  } while (0)
  if (three) {
    // the score kernel addresses the Pk rows of a batch row and the k_u rows of a head with 32-bit byte offsets when it
    // loads them straight into LDS
    const bool pk3 = pkl && ((int64_t)a.S * a.spk_s + a.Rk) * 2 < ((int64_t)1 << 32) && ((int64_t)a.Dh * a.ldku + a.Rk) * 2 < ((int64_t)1 << 32);
    // one query head per kv head over caches shared by the heads: two heads per workgroup read every Pk row once
    const bool pair = rep == 1 && (a.Hk % 2) == 0 && a.spk_h == 0 && pk3 && per >= 128;
    if (pair) {
#define FSVD_RD_LAUNCH_PAIR(KS_)                                                                                                    \
  do {                                                                                                                              \
    constexpr int lds = RankPairLds<KS_>::kBytes;                                                                                   \
    static bool granted = false;                                                                                                    \
    if (!granted) {                                                                                                                 \
      hipError_t ea = hipFuncSetAttribute(reinterpret_cast<const void*>(&rank_scores_pair_kernel<DT, KS_>),                             \
                                          hipFuncAttributeMaxDynamicSharedMemorySize, lds);                                         \
      if (ea != hipSuccess) { set_last_error("%s: cannot reserve %d bytes of LDS: %s", fn, lds, hipGetErrorString(ea)); return kErrLaunch; } \
      granted = true;                                                                                                               \
    }                                                                                                                               \
    hipLaunchKernelGGL((rank_scores_pair_kernel<DT, KS_>), dim3(a.nsplit, a.Hk / 2, a.B), dim3(kRdPairThreads), lds, st, a3);           \
  } while (0)
      if (per >= 256) FSVD_RD_LAUNCH_PAIR(4); else FSVD_RD_LAUNCH_PAIR(2);
#undef FSVD_RD_LAUNCH_PAIR
    } else
    if (rep % 4 == 0) { if (pk3) FSVD_RD_LAUNCH_SC(4, 1, true, a.Hk * (rep / 4)); else FSVD_RD_LAUNCH_SC(4, 1, false, a.Hk * (rep / 4)); }
    else if (rep % 2 == 0) { if (pk3) FSVD_RD_LAUNCH_SC(2, 2, true, a.Hk * (rep / 2)); else FSVD_RD_LAUNCH_SC(2, 2, false, a.Hk * (rep / 2)); }
    else if (per >= 256) { if (pk3) FSVD_RD_LAUNCH_SC(1, 4, true, a.Hk * rep); else FSVD_RD_LAUNCH_SC(1, 4, false, a.Hk * rep); }
    else { if (pk3) FSVD_RD_LAUNCH_SC(1, 2, true, a.Hk * rep); else FSVD_RD_LAUNCH_SC(1, 2, false, a.Hk * rep); }
    hipError_t e3 = hipGetLastError();
    if (e3 != hipSuccess) { set_last_error("%s: score launch failed: %s", fn, hipGetErrorString(e3)); return kErrLaunch; }
    hipLaunchKernelGGL(rank_decode_softmax_kernel<DT>, dim3(a.nsplit, a.H, a.B), block, 0, st, a3);
    const int mt = a.H > 16 ? 2 : 1;
    const dim3 gpv((a.Rv + 127) / 128, a.nsplit * ((a.H + 16 * mt - 1) / (16 * mt)), a.B);
    if (mt == 2) hipLaunchKernelGGL((rank_decode_pv_kernel<DT, 2>), gpv, block, 0, st, a3);
    else hipLaunchKernelGGL((rank_decode_pv_kernel<DT, 1>), gpv, block, 0, st, a3);
    e3 = hipGetLastError();
    if (e3 != hipSuccess) { set_last_error("%s: softmax / accumulation launch failed: %s", fn, hipGetErrorString(e3)); return kErrLaunch; }
  } else
  if (rep % 4 == 0) FSVD_RD_LAUNCH(4, 1, a.Hk * (rep / 4));
  else if (rep % 2 == 0) {
    if (ks >= 2) FSVD_RD_LAUNCH(2, 2, a.Hk * (rep / 2));
    else FSVD_RD_LAUNCH(2, 1, a.Hk * (rep / 2));
  } else {
    if (ks >= 2) FSVD_RD_LAUNCH(1, 2, a.Hk * rep);
    else FSVD_RD_LAUNCH(1, 1, a.Hk * rep);
  }
#undef FSVD_RD_LAUNCH_T
#undef FSVD_RD_LAUNCH_SC
#undef FSVD_RD_LAUNCH
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("%s: stage 1 launch failed: %s", fn, hipGetErrorString(e)); return kErrLaunch; }
  // head-dimension slices: enough workgroups for two per compute unit, at most eight per head (16 rows each)
  int dz = 1;
  while (dz < 8 && (int64_t)a.H * a.B * dz < 512) dz *= 2;
  hipLaunchKernelGGL(rank_decode_merge_kernel<DT>, dim3(a.H, a.B, dz), block, 0, st, a);
  e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("%s: stage 2 launch failed: %s", fn, hipGetErrorString(e)); return kErrLaunch; }
  return kOk;
}

int launch_rank_decode(const RankDecodeArgs& a, hipStream_t st) {
  if (a.dt != 0 && a.dt != 1) { set_last_error("fsvd_attn_decode_rankkv: dtype code %d (bf16 = 0 and fp16 = 1 are served)", a.dt); return kErrBadDtype; }
  return a.dt == 1 ? launch_rank_decode_t<1>(a, st) : launch_rank_decode_t<0>(a, st);
}

// One token's rank coefficients into the caches: cache[b, positions[b], :] = row b (16-byte pieces; a row whose position
// is outside [0, S) is dropped).  One launch instead of an index tensor and two scatters.
__global__ __launch_bounds__(256) void rankkv_append_kernel(const uint16_t* pk, int64_t ldpk, const uint16_t* pv, int64_t ldpv,
                                                            uint16_t* pkc, int64_t spk_b, int64_t spk_s, uint16_t* pvc, int64_t spv_b,
                                                            int64_t spv_s, const int32_t* positions, int S, int Rk, int Rv) {
  const int b = blockIdx.x, pos = positions[b];
  if (pos < 0 || pos >= S) return;
  const int nk = Rk / 8, nv = Rv / 8;
  for (int i = threadIdx.x; i < nk + nv; i += blockDim.x) {
    if (i < nk)
      *reinterpret_cast<u32x4_t*>(pkc + (int64_t)b * spk_b + (int64_t)pos * spk_s + i * 8) = *reinterpret_cast<const u32x4_t*>(pk + (int64_t)b * ldpk + i * 8);
    else
      *reinterpret_cast<u32x4_t*>(pvc + (int64_t)b * spv_b + (int64_t)pos * spv_s + (i - nk) * 8) = *reinterpret_cast<const u32x4_t*>(pv + (int64_t)b * ldpv + (i - nk) * 8);
  }
}
int launch_rankkv_append(const uint16_t* pk, int64_t ldpk, const uint16_t* pv, int64_t ldpv, uint16_t* pkc, int64_t spk_b, int64_t spk_s,
                         uint16_t* pvc, int64_t spv_b, int64_t spv_s, const int32_t* positions, int B, int S, int Rk, int Rv, hipStream_t st) {
  hipLaunchKernelGGL(rankkv_append_kernel, dim3(B), dim3(256), 0, st, pk, ldpk, pv, ldpv, pkc, spk_b, spk_s, pvc, spv_b, spv_s, positions, S, Rk, Rv);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("fsvd_rankkv_append: launch failed: %s", hipGetErrorString(e)); return kErrLaunch; }
  return kOk;
}

}  // namespace fsvd
