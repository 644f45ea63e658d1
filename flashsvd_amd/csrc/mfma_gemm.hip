// Prefill projections: y[M, N] = epilogue(x[M, K] . W[N, K]^T) for 128 rows and more, on the matrix cores.
//
// Both operands are K-contiguous, which is the layout V_MFMA_F32_16X16X32_BF16 wants for its two inputs (each lane
// holds 8 consecutive k of one row).  A workgroup of four or eight waves owns a 128 x 128, 128 x 64 or 64 x 64 output
// tile (32 x 64 below 128 rows) — the launcher picks by how many tiles the problem has for 256 compute units — and walks
// K in steps of 32, 64 or 128 through two LDS stages (the 16-byte pieces of a row swizzled so that the fragment reads of
// 16 consecutive rows fall on different banks).  Two ways to fill a stage: global loads that run two to four steps
// ahead in registers and are written to the idle stage one step before their products (few workgroups per compute
// unit, long K: latency-bound), or loads that write LDS themselves one step ahead (no staging registers, no LDS write
// instructions; pays when two or three workgroups share a compute unit).  The products are W . x^T, so a lane of the
// accumulator owns four consecutive output columns of one row (8-byte epilogue accesses).  Epilogue as in the vector
// kernels: bias, ONE rounding to bf16, residual — or, for the gate / up pair, SwiGLU in either rounding mode — or the
// head expansion of the prompt pass (RoPE, store into the query buffer or the cache rows).  Few tiles or a very long K:
// K split over workgroups, partial tiles added in a fixed order by the last arrival.
#include <algorithm>

#include "common.hpp"
#include "kernels.hpp"

namespace fsvd {

typedef float gm_f32x4_t __attribute__((ext_vector_type(4)));

constexpr int kGT4 = 256;           // threads of the four-wave form: 2 x 2 waves
constexpr int kGBK = 64;            // K per step (the small tile takes 128 when K allows: half as many barriers)

// WT: 16 x 16 accumulator tiles per wave and dimension: 4 -> 128 x 128 per workgroup, 2 -> 64 x 64 (problems with
// few output tiles, where more workgroups matter more than reuse)
// EXPAND: the head-expansion form of the prefill (y = P . u^T per head, then rotate-half RoPE at the token's position
// and a store into the query buffer or the cache rows): a column tile is one 128-wide head, and a wave takes columns
// [32 wn, 32 wn + 32) and [64 + 32 wn, 64 + 32 wn + 32) of it so that d and d + 64 of a rotation pair sit in one lane
struct ExpandEpi {
  const uint16_t* cos; const uint16_t* sin; int rope_len;
  const int32_t* positions;
  int M;                                   // tokens per batch row (x row r = batch r / M, token r % M)
  int64_t sp_b, sp_m;                      // strides of the coefficient rows
  int64_t sy_b, sy_m, sy_h;                // destination strides
  int dst_by_position, dst_rows;
};

// NW: waves per workgroup.  4: a wave owns a 16 WTM x 16 WT block of the output tile (both matrices of the gate / up
// pair).  8, pair (128 x 128 only): waves 0-3 accumulate the gate matrix and waves 4-7 the up matrix of the same
// blocks, which halves the accumulators per wave (two waves per SIMD instead of one); the up halves cross to their
// gate partners through LDS once, before the SwiGLU epilogue.  8, single matrix: waves 4-7 take the second half of the
// k slices of every step and hand their sums to waves 0-3 through LDS at the end.
// PF > 0: register sets in flight; PF < 0: loads straight into LDS with -PF stages.
template <int DT, bool DUAL, int WTM, int WT, int PF, bool EXPAND, int BK, int NW>
__device__ __forceinline__ void gemm_tiles_body(const MfmaArgs& a, const ExpandEpi& ep, const int tile_m, const int tile_n) {
  typedef E16<DT> E;
  typedef typename E::frag_t frag_t;
  static_assert(!EXPAND || (!DUAL && WT == 4), "head expansion takes whole 128-wide heads");
  static_assert(NW == 4 || (NW == 8 && DUAL && WT == 4 && WTM == 4) || (NW == 8 && !DUAL && !EXPAND && BK >= 64),
                "eight waves: the split form of the 128 x 128 pair tile, or two halves of every K step of a single matrix");
  constexpr int kGT = NW * 64;
  constexpr bool SPLIT = NW == 8 && DUAL;
  // single matrix, eight waves: waves 4-7 take the second half of the k slices of every step and hand their sums to
  // waves 0-3 at the end (a tile that has a compute unit to itself then still runs two waves per SIMD)
  constexpr bool KHALF = NW == 8 && !DUAL;
  constexpr bool DTL = PF < 0;            // global loads write the LDS stages themselves (no register sets), -PF stages
  constexpr int PFR = DTL ? 1 : PF;
  constexpr int NS = DTL ? -PF : 2;       // LDS stages
  constexpr int NM = DUAL ? 2 : 1;
  constexpr int NMA = SPLIT ? 1 : NM;     // accumulator sets per wave
  constexpr int kGLd = BK;                // LDS row stride in elements: no padding, the 16-byte pieces of a row are swizzled
  constexpr int CPR = BK / 8;             // 16-byte pieces per tile row
  constexpr int NPX = 32 * WTM * CPR / kGT; // pieces per thread of an x tile
  constexpr int NP = 32 * WT * CPR / kGT;   // ... of a W tile
  constexpr int kGBM = 32 * WTM, kGBN = 32 * WT;
  extern __shared__ __align__(16) unsigned char gm_smem[];
  // [stage][operand: x0, (x1), W0, (W1)][128 rows][kGLd]
  uint16_t* lds = reinterpret_cast<uint16_t*>(gm_smem);
  constexpr int kTileX = kGBM * kGLd, kTileW = kGBN * kGLd;   // elements per operand tile
  constexpr int kStage = NM * (kTileX + kTileW);
  const int tid = threadIdx.x, wave = (tid >> 6) & 3, lane = tid & 63, lr = lane & 15, lg = lane >> 4;
  const int mat = NW == 8 ? (tid >> 8) : 0;   // eight waves: which matrix of the pair / which half of the k slices
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = tile_m * kGBM, n0 = tile_n * kGBN;
  // this workgroup's share of the K steps (all of them unless K is split over gridDim.z)
  const int ksteps_all = a.K / BK;
  const int kper = (ksteps_all + (int)gridDim.z - 1) / (int)gridDim.z;
  const int kbeg = min((int)blockIdx.z * kper, ksteps_all);
  const int ksteps = max(1, min(kper, ksteps_all - kbeg));   // a share past the end re-reads the last step and adds zero
  const bool kdead = kbeg >= ksteps_all;

  // global -> register staging: a tile row is CPR 16-byte pieces; NP pieces per thread and operand
  constexpr int RPP = kGT / CPR;                      // rows covered by one pass of the workgroup
  const int ld_row = tid / CPR, ld_chunk = tid % CPR; // rows ld_row + RPP * j, j = 0..NP-1
  // LDS swizzle: piece c of row r sits at piece c ^ (r % CPR).  A 16-byte LDS read is served 16 lanes a cycle, in the
  // groups {0-3, 12-15, 20-27} and {4-11, 16-19, 28-31} of each half wave; with this placement the fragment reads
  // below (lane = row % 16 + 16 * piece) touch every bank once per group, which row padding of 16 bytes does not
  // achieve (two lanes per bank, half the read rate).  RPP and the fragment row bases are multiples of CPR, so the
  // swizzle term of a thread never changes.
  // (Rows of 64 bytes, K steps of 32: four rows span the banks once, and the term is (-(r / 4)) % 4 instead.)
  static_assert(RPP % 16 == 0 && CPR >= 4 && CPR <= 16, "swizzle term must be constant per thread");
  const auto swz = [](int r) { return CPR == 4 ? ((-(r >> 2)) & 3) : r % CPR; };
  const int st_chunk = ld_chunk ^ swz(ld_row);
  // direct form: lane i of a load instruction lands at 16 i bytes past the instruction's LDS base, i.e. at piece
  // ld_chunk of its row, so it fetches the piece that belongs there
  const int g_chunk = DTL ? st_chunk : ld_chunk;
  const int fr_hi = swz(lr) & ~3, fr_lo = lg ^ (swz(lr) & 3);   // fragment piece kk*4 + lg -> ((kk*4) ^ fr_hi) + fr_lo
  const uint16_t* gx[NM][NPX];
  const uint16_t* gw[NM][NP];
#pragma unroll
  for (int j = 0; j < NPX; ++j) {
    const int64_t xr = min(m0 + ld_row + RPP * j, a.B - 1);
    if (EXPAND) gx[0][j] = a.x + (xr / ep.M) * ep.sp_b + (xr % ep.M) * ep.sp_m + g_chunk * 8;
    else gx[0][j] = a.x + xr * a.ldx + g_chunk * 8;
    if (DUAL) gx[NM - 1][j] = a.x + xr * a.ldx + a.up_off + g_chunk * 8;
  }
#pragma unroll
  for (int j = 0; j < NP; ++j) {
    const int64_t wr = min(n0 + ld_row + RPP * j, a.N - 1);
    gw[0][j] = a.W + wr * a.ldw + g_chunk * 8;
    if (DUAL) gw[NM - 1][j] = a.W2 + wr * a.ldw + g_chunk * 8;
  }
  // PF register sets hold the global loads of the next PF steps (set s % PF belongs to step s); a set is written
  // to the idle LDS stage one step before its products and refilled at once with the loads of step s + PF
  u32x4_t rx[PFR][NM][NPX], rw[PFR][NM][NP];
  auto load_regs = [&](int set, int ks) {
    const int k = min(kbeg + min(ks, ksteps - 1), ksteps_all - 1) * BK;   // past the end: a valid address, never used
#pragma unroll
    for (int m = 0; m < NM; ++m) {
#pragma unroll
      for (int j = 0; j < NPX; ++j) rx[set][m][j] = *reinterpret_cast<const u32x4_t*>(gx[m][j] + k);
#pragma unroll
      // plain loads: the other row tiles resident on this XCD read the same W tile out of its L2 (a streaming hint
      // gives the lines up early: 10..25 % slower at 512 rows and more)
      for (int j = 0; j < NP; ++j) rw[set][m][j] = *reinterpret_cast<const u32x4_t*>(gw[m][j] + k);
    }
  };
  auto store_lds = [&](int set, int stage) {
    uint16_t* base = lds + stage * kStage;
#pragma unroll
    for (int m = 0; m < NM; ++m) {
#pragma unroll
      for (int j = 0; j < NPX; ++j) *reinterpret_cast<u32x4_t*>(base + m * kTileX + (ld_row + RPP * j) * kGLd + st_chunk * 8) = rx[set][m][j];
#pragma unroll
      for (int j = 0; j < NP; ++j)
        *reinterpret_cast<u32x4_t*>(base + NM * kTileX + m * kTileW + (ld_row + RPP * j) * kGLd + st_chunk * 8) = rw[set][m][j];
    }
  };

  typedef const __attribute__((address_space(1))) void* gm_gptr_t;
  typedef __attribute__((address_space(3))) void* gm_lptr_t;
  const auto issue_direct = [&](int stage, int ks) {
    const int k = min(kbeg + min(ks, ksteps - 1), ksteps_all - 1) * BK;
    uint16_t* sb = lds + stage * kStage + ((tid >> 6) * (64 / CPR)) * kGLd;   // this wave's rows of a pass
#pragma unroll
    for (int m = 0; m < NM; ++m) {
#pragma unroll
      for (int j = 0; j < NPX; ++j)
        __builtin_amdgcn_global_load_lds((gm_gptr_t)(gx[m][j] + k), (gm_lptr_t)(sb + m * kTileX + RPP * j * kGLd), 16, 0, 0);
#pragma unroll
      for (int j = 0; j < NP; ++j)
        __builtin_amdgcn_global_load_lds((gm_gptr_t)(gw[m][j] + k), (gm_lptr_t)(sb + NM * kTileX + m * kTileW + RPP * j * kGLd), 16, 0, 0);
    }
  };

  gm_f32x4_t acc[NMA][WTM][WT];
#pragma unroll
  for (int m = 0; m < NMA; ++m)
#pragma unroll
    for (int i = 0; i < WTM; ++i)
#pragma unroll
      for (int j = 0; j < WT; ++j) acc[m][i][j] = gm_f32x4_t{0.f, 0.f, 0.f, 0.f};

  // direct form: the loads of step s + NS - 1 are issued during step s; all but the newest NS - 2 groups of kLd loads
  // have to be complete before the barrier that opens the next stage
  constexpr int kLd = NM * (NPX + NP), kOpen = (NS - 2) * kLd;
  static_assert(kOpen < 64, "vmcnt holds six bits");
  constexpr int kWaitOpen = (kOpen & 15) | (7 << 4) | (15 << 8) | ((kOpen >> 4) << 14);
  if (DTL) {
#pragma unroll
    for (int s0 = 0; s0 < NS - 1; ++s0) issue_direct(s0, s0);
    __builtin_amdgcn_s_waitcnt(kWaitOpen);
  } else {
#pragma unroll
    for (int u = 0; u < PFR; ++u) load_regs(u, u);
    store_lds(0, 0);
    load_regs(0, PFR);
  }
  __syncthreads();
  for (int ks0 = 0; ks0 < ksteps; ks0 += PFR) {
#pragma unroll
    for (int u = 0; u < PFR; ++u) {
      const int ks = ks0 + u;
      if (ks >= ksteps) break;
      const uint16_t* base = lds + (ks % NS) * kStage;
      // The step as Q blocks of WTM x WT products (k slice kk of matrix ma).  The fragments of block q + 1 are read
      // while block q multiplies, and the last block, which has nothing left to read, carries the LDS writes of the
      // next stage and the global loads that refill their registers: the other stage was last read before the
      // barrier that ended step ks - 1, and past the last step both are harmless (clamped addresses, a dead stage).
      constexpr int Q = KHALF ? BK / 64 : (BK / 32) * NMA;
      frag_t fx[2][WTM], fw[2][WT];
      const auto load_frags = [&](int q, int set) {
        const int kk = KHALF ? mat * (BK / 64) + q : q / NMA, m = SPLIT ? mat : (KHALF ? 0 : q % NMA);
        const int fcol = (((kk * 4) ^ fr_hi) + fr_lo) * 8;
#pragma unroll
        for (int i = 0; i < WTM; ++i)
          fx[set][i] = *reinterpret_cast<const frag_t*>(base + m * kTileX + (wm * 16 * WTM + i * 16 + lr) * kGLd + fcol);
#pragma unroll
        for (int i = 0; i < WT; ++i) {
          const int wrow = EXPAND ? (i < 2 ? wn * 32 + i * 16 : 64 + wn * 32 + (i - 2) * 16) : wn * 16 * WT + i * 16;
          fw[set][i] = *reinterpret_cast<const frag_t*>(base + NM * kTileX + m * kTileW + (wrow + lr) * kGLd + fcol);
        }
      };
      load_frags(0, 0);
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        if (DTL && q == 0) issue_direct((ks + NS - 1) % NS, ks + NS - 1);
        if (q + 1 < Q) {
          load_frags(q + 1, (q + 1) & 1);
        } else if (!DTL) {
          store_lds((u + 1) % PFR, (ks + 1) & 1);
          load_regs((u + 1) % PFR, ks + 1 + PFR);
        }
#pragma unroll
        for (int i = 0; i < WTM; ++i)
#pragma unroll
          for (int j = 0; j < WT; ++j)
            acc[q % NMA][i][j] = E::mfma(fw[q & 1][j], fx[q & 1][i], acc[q % NMA][i][j]);
        // issue order: memory instructions spread between the products instead of ahead of them
        constexpr int kMf = WTM * WT;
        if (q + 1 < Q) {
          constexpr int kRd = WTM + WT, kPer = kMf / kRd > 0 ? kMf / kRd : 1;
#pragma unroll
          for (int n = 0; n < kRd; ++n) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);     // one LDS read
            __builtin_amdgcn_sched_group_barrier(0x008, kPer, 0);  // products
          }
        } else if (!DTL) {
          constexpr int kWr = NM * (NPX + NP), kPer = kMf / kWr > 0 ? kMf / kWr : 1;
#pragma unroll
          for (int n = 0; n < kWr; ++n) {
            __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);     // one LDS write
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);     // one global load
            __builtin_amdgcn_sched_group_barrier(0x008, kPer, 0);
          }
        }
      }
      if (DTL) __builtin_amdgcn_s_waitcnt(kWaitOpen);   // this wave's pieces of the next stage have landed
      __syncthreads();
    }
  }

  if (KHALF) {
    gm_f32x4_t* ex = reinterpret_cast<gm_f32x4_t*>(gm_smem);     // [WTM*WT][256] 16-byte words, inside the stages
    __syncthreads();                                             // every wave has finished reading the last stage
    if (mat == 1) {
#pragma unroll
      for (int i = 0; i < WTM; ++i)
#pragma unroll
        for (int j = 0; j < WT; ++j) ex[(i * WT + j) * 256 + (tid & 255)] = acc[0][i][j];
    }
    __syncthreads();
    if (mat == 0) {
#pragma unroll
      for (int i = 0; i < WTM; ++i)
#pragma unroll
        for (int j = 0; j < WT; ++j) acc[0][i][j] += ex[(i * WT + j) * 256 + (tid & 255)];
    }
  }
  const bool writer = !KHALF || mat == 0;   // waves 4-7 of the halved form keep the barriers below company and store nothing
  // K split: park the partial tile (thread-major 16-byte words, coalesced), count arrivals; the last workgroup of a
  // tile adds all partials in split order (its own included, so the sum does not depend on who came last)
  if (WTM <= 2 && gridDim.z > 1) {         // only the 32- and 64-row tiles are ever launched with a split
    constexpr int WPT = NMA * WTM * WT;                          // 16-byte words per thread
    const int tile = blockIdx.y * gridDim.x + blockIdx.x;
    gm_f32x4_t* part = reinterpret_cast<gm_f32x4_t*>(a.ws_part) + (size_t)tile * gridDim.z * WPT * kGT;
    gm_f32x4_t* mine = part + (size_t)blockIdx.z * WPT * kGT;
    // write-through agent-scope stores (they do not stay dirty in this XCD's L2), all of them acknowledged before the
    // arrival is counted; the reader below uses agent-scope loads, which do not look into its own L2.  No fence: a
    // release or acquire fence per workgroup writes back / empties a whole L2 under the weight stream of the others
#pragma unroll
    for (int m = 0; m < NMA; ++m)
#pragma unroll
      for (int i = 0; i < WTM; ++i)
#pragma unroll
        for (int j = 0; j < WT; ++j) {
          if (!writer) break;
          const gm_f32x4_t v = kdead ? gm_f32x4_t{0.f, 0.f, 0.f, 0.f} : acc[m][i][j];
          unsigned long long* dst = reinterpret_cast<unsigned long long*>(mine + ((m * WTM + i) * WT + j) * kGT + tid);
          __hip_atomic_store(dst, ((unsigned long long)__float_as_uint(v[1]) << 32) | __float_as_uint(v[0]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(dst + 1, ((unsigned long long)__float_as_uint(v[3]) << 32) | __float_as_uint(v[2]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    int* flag = reinterpret_cast<int*>(gm_smem);
    if (tid == 0) {
      const int prev = atomicAdd(a.ws_count + tile, 1);
      const int last = prev == (int)gridDim.z - 1;
      if (last) a.ws_count[tile] = 0;                            // ready for the next launch
      *flag = last;
    }
    __syncthreads();
    if (*flag == 0 || !writer) return;
    // the shares are added in split order; the loads of several shares are in flight at once (each comes from beyond
    // this XCD's L2, and one share per round trip made the reduction the longest part of a narrow projection)
    constexpr int ZC = WPT <= 2 ? 8 : (WPT <= 4 ? 4 : 2);
#pragma unroll
    for (int m = 0; m < NMA; ++m)
#pragma unroll
      for (int i = 0; i < WTM; ++i)
#pragma unroll
        for (int j = 0; j < WT; ++j) acc[m][i][j] = gm_f32x4_t{0.f, 0.f, 0.f, 0.f};
    for (int z0 = 0; z0 < (int)gridDim.z; z0 += ZC) {
      unsigned long long lo[ZC][WPT], hi[ZC][WPT];
#pragma unroll
      for (int u = 0; u < ZC; ++u) {
        const int z = min(z0 + u, (int)gridDim.z - 1);
#pragma unroll
        for (int w = 0; w < WPT; ++w) {
          const unsigned long long* src = reinterpret_cast<const unsigned long long*>(part + (size_t)z * WPT * kGT + w * kGT + tid);
          lo[u][w] = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          hi[u][w] = __hip_atomic_load(src + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
#pragma unroll
      for (int u = 0; u < ZC; ++u) {
        if (z0 + u >= (int)gridDim.z) break;
#pragma unroll
        for (int m = 0; m < NMA; ++m)
#pragma unroll
          for (int i = 0; i < WTM; ++i)
#pragma unroll
            for (int j = 0; j < WT; ++j) {
              const int w = (m * WTM + i) * WT + j;
              acc[m][i][j] += gm_f32x4_t{__uint_as_float((uint32_t)lo[u][w]), __uint_as_float((uint32_t)(lo[u][w] >> 32)),
                                         __uint_as_float((uint32_t)hi[u][w]), __uint_as_float((uint32_t)(hi[u][w] >> 32))};
            }
      }
    }
  }
  if (!writer) return;
  // split pair: the up accumulators travel to the gate wave of the same block (same lane, same tile indices)
  gm_f32x4_t upv[SPLIT ? WTM : 1][SPLIT ? WT : 1];
  if (SPLIT) {
    gm_f32x4_t* ex = reinterpret_cast<gm_f32x4_t*>(gm_smem);     // [WTM*WT][256] 16-byte words, at most half of the stages
    __syncthreads();                                             // every wave has finished reading the last stage
    if (mat == 1) {
#pragma unroll
      for (int i = 0; i < WTM; ++i)
#pragma unroll
        for (int j = 0; j < WT; ++j) ex[(i * WT + j) * 256 + (tid & 255)] = acc[0][i][j];
    }
    __syncthreads();
    if (mat == 1) return;
#pragma unroll
    for (int i = 0; i < WTM; ++i)
#pragma unroll
      for (int j = 0; j < WT; ++j) upv[i][j] = ex[(i * WT + j) * 256 + (tid & 255)];
  }
  // The products are taken as W . x^T (W fragment as the first operand), so element e of lane l of tile (i, j) is row
  // m = i*16 + l%16 of x and column n = j*16 + (l/16)*4 + e of W: a lane owns four consecutive columns of one row and
  // stores them with one 8-byte write (one 2-byte write each when the destination is not 8-byte aligned)
  const auto al8 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7) == 0; };
#pragma unroll
  for (int i = 0; i < WTM; ++i) {
    const int m = m0 + wm * 16 * WTM + i * 16 + lr;
    if (m >= a.B) continue;
    if (EXPAND) {
      const int b = m / ep.M, t = m - b * ep.M;
      const int pos = (ep.positions ? ep.positions[b] : 0) + t;
      const int slot = ep.dst_by_position ? pos : t;
      if (slot < 0 || slot >= ep.dst_rows) continue;   // outside the destination: dropped
      const int head = tile_n;
      uint16_t* dst = a.y + (int64_t)b * ep.sy_b + (int64_t)slot * ep.sy_m + (int64_t)head * ep.sy_h;
      const int tp = min(max(pos, 0), ep.rope_len - 1);
      const bool dst8 = al8(dst), tab8 = ep.cos && al8(ep.cos) && al8(ep.sin);
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int d0 = wn * 32 + j * 16 + lg * 4;
        float c[4], sn[4];
        if (ep.cos) {
          if (tab8) {
            const u32x2_t cw = *reinterpret_cast<const u32x2_t*>(ep.cos + (int64_t)tp * 64 + d0);
            const u32x2_t sw = *reinterpret_cast<const u32x2_t*>(ep.sin + (int64_t)tp * 64 + d0);
            c[0] = E::lo(cw.x); c[1] = E::hi(cw.x); c[2] = E::lo(cw.y); c[3] = E::hi(cw.y);
            sn[0] = E::lo(sw.x); sn[1] = E::hi(sw.x); sn[2] = E::lo(sw.y); sn[3] = E::hi(sw.y);
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              c[e] = E::val(ep.cos[(int64_t)tp * 64 + d0 + e]);
              sn[e] = E::val(ep.sin[(int64_t)tp * 64 + d0 + e]);
            }
          }
        }
        uint32_t o0[4], o1[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int d = d0 + e;
          float x0 = acc[0][i][j][e], x1 = acc[0][i][j + 2][e];
          if (a.bias) { x0 += E::val(a.bias[head * 128 + d]); x1 += E::val(a.bias[head * 128 + d + 64]); }
          x0 = E::rnd(x0);                          // the projection's own rounding point
          x1 = E::rnd(x1);
          if (ep.cos) {                                 // eager bf16 arithmetic, one rounding per op
            const float r0 = E::rnd(E::rnd(x0 * c[e]) - E::rnd(x1 * sn[e]));
            const float r1 = E::rnd(E::rnd(x1 * c[e]) + E::rnd(x0 * sn[e]));
            x0 = r0; x1 = r1;
          }
          o0[e] = E::bits(x0);
          o1[e] = E::bits(x1);
        }
        if (dst8) {
          *reinterpret_cast<u32x2_t*>(dst + d0) = u32x2_t{o0[0] | (o0[1] << 16), o0[2] | (o0[3] << 16)};
          *reinterpret_cast<u32x2_t*>(dst + d0 + 64) = u32x2_t{o1[0] | (o1[1] << 16), o1[2] | (o1[3] << 16)};
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) { dst[d0 + e] = (uint16_t)o0[e]; dst[d0 + 64 + e] = (uint16_t)o1[e]; }
        }
      }
      continue;
    }
    uint16_t* yrow = a.y + (int64_t)m * a.ldy;
    const uint16_t* rrow = a.res ? a.res + (int64_t)m * a.ldres : nullptr;
    const bool y8 = al8(yrow), r8 = rrow && al8(rrow);
#pragma unroll
    for (int j = 0; j < WT; ++j) {
      const int nb = n0 + wn * 16 * WT + j * 16 + lg * 4;
      if (nb >= a.N) continue;
      const bool whole = nb + 3 < a.N;
      float r[4] = {0.f, 0.f, 0.f, 0.f};
      if (!DUAL && rrow) {
        if (whole && r8) {
          const u32x2_t rw = *reinterpret_cast<const u32x2_t*>(rrow + nb);
          r[0] = E::lo(rw.x); r[1] = E::hi(rw.x); r[2] = E::lo(rw.y); r[3] = E::hi(rw.y);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (nb + e < a.N) r[e] = E::val(rrow[nb + e]);
        }
      }
      uint32_t o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v0 = acc[0][i][j][e];
        float v;
        if (DUAL) {
          float v1 = SPLIT ? upv[SPLIT ? i : 0][SPLIT ? j : 0][e] : acc[NMA - 1][i][j][e];
          if (a.mode == 0) {
            v0 = E::rnd(v0);
            v1 = E::rnd(v1);
            v = E::rnd(E::rnd(silu_f32(v0)) * v1);
          } else {
            v = E::rnd((v0 * (1.0f / (1.0f + expf(-v0)))) * v1);
          }
        } else {
          if (a.bias && nb + e < a.N) v0 += E::val(a.bias[nb + e]);
          v = E::rnd(v0);
          if (rrow) v = E::rnd(r[e] + v);
        }
        o[e] = E::bits(v);
      }
      if (whole && y8) {
        *reinterpret_cast<u32x2_t*>(yrow + nb) = u32x2_t{o[0] | (o[1] << 16), o[2] | (o[3] << 16)};
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (nb + e < a.N) yrow[nb + e] = (uint16_t)o[e];
      }
    }
  }
}

// every XCD takes one contiguous run of tiles, ordered in bands of eight row tiles walked column by column, so that
// the workgroups resident on an XCD at one time share a few x tiles and a few W tiles in its L2
__device__ __forceinline__ void tile_of_workgroup(int NT, int MT, int& tile_m, int& tile_n) {
  const int t = xcd_run_index(blockIdx.y * NT + blockIdx.x, NT * MT);
  const int band = t / (8 * NT), tb = t - band * 8 * NT;
  const int bh = min(8, MT - band * 8);
  tile_n = tb / bh;
  tile_m = band * 8 + tb - tile_n * bh;
}

template <int DT, bool DUAL, int WTM, int WT, int PF, bool EXPAND, int BK, int NW>
__global__ __launch_bounds__(NW * 64, NW == 8 ? 1 : 2) void gemm_tiles_kernel(MfmaArgs a, ExpandEpi ep) {
  int tile_m, tile_n;
  tile_of_workgroup(gridDim.x, gridDim.y, tile_m, tile_n);
  gemm_tiles_body<DT, DUAL, WTM, WT, PF, EXPAND, BK, NW>(a, ep, tile_m, tile_n);
}

// up to three head expansions of the same token rows (q, k, v of a prompt pass) in one launch: column tile = one head
// of one of them.  At 512 rows a single expansion has one workgroup per compute unit and waits on its own loads; the
// three together give every compute unit three.
struct ExpandBatch { MfmaArgs a[3]; ExpandEpi ep[3]; int first_head[4]; };
template <int DT, int WTM>
__global__ __launch_bounds__(kGT4, 2) void expand_multi_kernel(ExpandBatch eb) {
  int tile_m, tile_n;
  tile_of_workgroup(gridDim.x, gridDim.y, tile_m, tile_n);
  const int k = tile_n >= eb.first_head[2] ? 2 : (tile_n >= eb.first_head[1] ? 1 : 0);
  gemm_tiles_body<DT, false, WTM, 4, 2, true, kGBK, 4>(eb.a[k], eb.ep[k], tile_m, tile_n - eb.first_head[k]);
}

bool gemm_tiles_apply(const MfmaArgs& a) {
  return a.B >= 128 && (a.K % kGBK) == 0 && (a.ldw % 8) == 0 && (a.ldx % 8) == 0 && (a.up_off % 8) == 0;
}

// K split for a grid of `tiles` workgroups: enough shares to give every compute unit two workgroups, at least four
// K steps per share, and only as many as the registered workspace holds (1 = no split)
static int fit_ksplit(int z, int64_t tiles, int ksteps, size_t floats_per_share, const SplitWorkspace& ws, int cap) {
  if (ws.part == nullptr || tiles > ws.ncount) return 1;
  z = std::min(z, std::min(cap, ksteps / 4));
  while (z > 1 && (size_t)tiles * z * floats_per_share > ws.part_floats) --z;
  return std::max(z, 1);
}
static int pick_ksplit(int64_t tiles, int ksteps, size_t floats_per_share, const SplitWorkspace& ws) {
  if (tiles >= 512) return 1;
  return fit_ksplit((int)((512 + tiles - 1) / tiles), tiles, ksteps, floats_per_share, ws, 16);
}
// 64 x 64 tiles of a prompt projection (128 rows and more): a split pays only where the unsplit launch leaves compute
// units idle (up to 128 tiles: two workgroups per tile-starved pair of compute units) or walks a very long K with at
// most two workgroups per compute unit (down_v of the 7B MLP, K = 11008).  Measured at 128..1024 rows with weights from
// HBM: o_v 18 -> 12..15 us, down_v 51 -> 25 (128 rows), 32 (256), 46 (512), 92 -> 76 (1024); everything else is as fast
// or faster unsplit.
static int pick_ksplit_prompt(int64_t tiles, int ksteps, int K, size_t floats_per_share, const SplitWorkspace& ws) {
  int z = 1;
  if (tiles <= 128) z = (int)((256 + tiles - 1) / tiles);
  if (K >= 8192 && tiles < 512) z = std::max(z, (int)((768 + tiles - 1) / tiles));
  return z > 1 ? fit_ksplit(z, tiles, ksteps, floats_per_share, ws, 8) : 1;
}

template <int DT, bool DUAL, int WTM, int WT, int BK, int NW = 4, int PFSEL = 99>
static int launch_gemm_tiles_t(const MfmaArgs& a0, hipStream_t st, const char* who) {
  static bool granted = false;
  constexpr int BM = 32 * WTM, BN = 32 * WT;
  constexpr int kGLd = BK;
  // register sets in flight: deep for the small single tile (few workgroups, latency-bound), two where a deeper
  // pipeline would cost a resident wave per SIMD
  constexpr int PF = PFSEL != 99 ? PFSEL : (!DUAL && WT == 2 && WTM == 2 && BK == 64) ? 4 : 2;
  const size_t lds = (size_t)(PF < 0 ? -PF : 2) * (DUAL ? 2 : 1) * (BM + BN) * kGLd * 2;
  if (lds > 64 * 1024 && !granted) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_tiles_kernel<DT, DUAL, WTM, WT, PF, false, BK, NW>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) { set_last_error("%s: cannot reserve %zu bytes of LDS: %s", who, lds, hipGetErrorString(e)); return kErrLaunch; }
    granted = true;
  }
  MfmaArgs a = a0;
  dim3 grid((a.N + BN - 1) / BN, (a.B + BM - 1) / BM, 1);
  const SplitWorkspace ws = split_workspace();
  constexpr size_t share = (size_t)(DUAL && NW == 4 ? 2 : 1) * WTM * WT * 4 * NW * 64;   // floats one workgroup parks
  // the 32-row tiles split K whenever that fills the chip; 64 x 64 prompt tiles only where measured to pay; larger
  // tiles never (parking and re-reading the partial tiles costs what the extra workgroups gain)
  if (WTM == 1) a.ksplit = pick_ksplit((int64_t)grid.x * grid.y, a.K / BK, share, ws);
  else if (WTM == 2 && !DUAL) a.ksplit = pick_ksplit_prompt((int64_t)grid.x * grid.y, a.K / BK, a.K, share, ws);
  else a.ksplit = 1;
  a.ws_part = ws.part;
  a.ws_count = ws.count;
  grid.z = a.ksplit;
  hipLaunchKernelGGL((gemm_tiles_kernel<DT, DUAL, WTM, WT, PF, false, BK, NW>), grid, dim3(NW * 64), lds, st, a, ExpandEpi{});
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("%s: launch failed: %s", who, hipGetErrorString(e)); return kErrLaunch; }
  return kOk;
}

template <int DT>
static int launch_gemm_tiles_dt(const MfmaArgs& a, bool dual, hipStream_t st, const char* who) {
  const int64_t big = (int64_t)((a.N + 127) / 128) * ((a.B + 127) / 128);
  // Forms by tile count (measured on the projections of the 7B shape at 128..4096 rows).  The pair kernel: the
  // eight-wave 128 x 128 form from two big tiles per compute unit on, else 64 x 64.  A single matrix: 128 x 128 from
  // 448 big tiles on, 128 x 64 from 256 on, else 64 x 64 — in K steps of 64 with a deep register pipeline when there
  // are more of those than the chip holds at once (320), in steps of 128 (half as many barriers) when there are fewer:
  // with one workgroup or less per compute unit and a long K only loads issued several steps ahead hide the latency.
  // The pair at four big tiles per compute unit and more: four waves with both accumulator sets, K steps of 32
  // loaded straight into LDS (two workgroups per compute unit; 243 -> 214 us at 2048 rows of the 7B MLP)
  if (dual && big >= 1024) return launch_gemm_tiles_t<DT, true, 4, 4, 32, 4, -2>(a, st, who);
  if (dual && big >= 512) return launch_gemm_tiles_t<DT, true, 4, 4, 64, 8>(a, st, who);
  // two and a half to four 64 x 128 tiles per compute unit: that tile, K steps of 32 straight into LDS, three
  // workgroups per compute unit (7B MLP at 512 rows 83 -> 77 us, at 768 rows 114 -> 110; slower outside this range)
  const int64_t wide = (int64_t)((a.N + 127) / 128) * ((a.B + 63) / 64);
  if (dual && wide >= 640 && wide <= 1100) return launch_gemm_tiles_t<DT, true, 2, 4, 32, 4, -2>(a, st, who);
  if (dual) return launch_gemm_tiles_t<DT, true, 2, 2, 64>(a, st, who);
  // a single matrix with more than one big tile per compute unit: loads straight into LDS, two stages (the second and
  // third workgroup of a compute unit cover the one-step load distance; 5..8 % faster than the register pipeline with
  // weights that come from HBM, and slower than it below these tile counts)
  // many tiles per compute unit (long prompts): 128 x 256 tiles, a wave on 64 x 128 of it -- a third fewer fragment
  // reads from LDS per product; K steps of 32 keep two workgroups per compute unit (16384 rows of the 7B shape at
  // ratio 0.8: 1..6 % faster per projection, same results bit for bit)
  if (big >= 2048) return launch_gemm_tiles_t<DT, false, 4, 8, 32, 4, -2>(a, st, who);
  if (big >= 448) return launch_gemm_tiles_t<DT, false, 4, 4, 64, 4, -2>(a, st, who);
  if (big >= 320) return launch_gemm_tiles_t<DT, false, 4, 2, 64, 4, -2>(a, st, who);
  // about one tile per compute unit: eight waves on a 128 x 128 or 128 x 64 tile, each half of them on half of the k
  // slices of a step, so that a workgroup alone on its compute unit still runs two waves per SIMD (rank projections at
  // 512 rows 36 -> 29 us, at 1024 rows 50 -> 43; down_v at 2048 rows 131 -> 109; with fewer tiles than ~0.6 per
  // compute unit the 64 x 64 tiles below win, with more the four-wave forms that share a compute unit)
  if (big >= 144 && big <= 256) return launch_gemm_tiles_t<DT, false, 4, 4, 64, 8>(a, st, who);
  if (big >= 256) return launch_gemm_tiles_t<DT, false, 4, 2, 64>(a, st, who);
  const int64_t half = (int64_t)((a.N + 63) / 64) * ((a.B + 127) / 128);
  if (half >= 160 && half <= 256 && (a.K % 128) == 0) return launch_gemm_tiles_t<DT, false, 4, 2, 128, 8>(a, st, who);
  const int64_t small = (int64_t)((a.N + 63) / 64) * ((a.B + 63) / 64);
  return (small < 320 && (a.K % 128) == 0) ? launch_gemm_tiles_t<DT, false, 2, 2, 128>(a, st, who) : launch_gemm_tiles_t<DT, false, 2, 2, 64>(a, st, who);
}

// 17..127 rows (batched decoding): 32-row tiles, 64 columns wide, K split over workgroups.  Needs the registered
// workspace (without the split a narrow projection would occupy a fraction of the compute units).  Up to 16 rows the
// wave-per-16-weight-rows kernel is as fast or faster (MLP of the 7B shape, 8 rows: 73 vs 79 us; 32 rows: 117 vs 75 us)
// unless the matrix has fewer than 128 of its 16-row tiles, one workgroup each (down_v of the 7B MLP, 1536 x 11008, at
// 8 rows: 22.6 us there, 17 us here).
bool gemm_rows_apply(const MfmaArgs& a) {
  const bool rows = a.B >= 17 || (a.B >= 3 && (a.N + 15) / 16 < 128);
  return rows && a.B < 128 && (a.K % kGBK) == 0 && (a.ldw % 8) == 0 && (a.ldx % 8) == 0 && (a.up_off % 8) == 0 &&
         split_workspace().part != nullptr;
}
int launch_gemm_tiles(const MfmaArgs& a, bool dual, hipStream_t st, const char* who) {
  return a.dt == 1 ? launch_gemm_tiles_dt<1>(a, dual, st, who) : launch_gemm_tiles_dt<0>(a, dual, st, who);
}
template <int DT>
static int launch_gemm_rows_dt(const MfmaArgs& a, bool dual, hipStream_t st, const char* who) {
  if (dual) return launch_gemm_tiles_t<DT, true, 1, 2, 64>(a, st, who);
  return (a.K % 128) == 0 ? launch_gemm_tiles_t<DT, false, 1, 2, 128>(a, st, who) : launch_gemm_tiles_t<DT, false, 1, 2, 64>(a, st, who);
}

int launch_gemm_rows(const MfmaArgs& a, bool dual, hipStream_t st, const char* who) {
  return a.dt == 1 ? launch_gemm_rows_dt<1>(a, dual, st, who) : launch_gemm_rows_dt<0>(a, dual, st, who);
}

// head expansion of the prefill on the tiled kernel: 128 token rows and more, head_dim 128, rank a multiple of 64,
// coefficients shared by the heads
bool expand_tiles_apply(const ExpandArgs& a) {
  return a.Dh == 128 && (int64_t)a.B * a.M >= 128 && (a.R % kGBK) == 0 && a.sp_h == 0 && (a.sp_b % 8) == 0 && (a.sp_m % 8) == 0 &&
         (a.ldu % 8) == 0;
}

template <int DT, int WTM>
static int launch_expand_tiles_t(const ExpandArgs& a, hipStream_t st) {
  const char* who = "fsvd_lowrank_expand_heads";
  static bool granted = false;
  constexpr int PF = 2;   // register pipeline (loads straight into LDS were slower here: 0.92 -> 1.03 ms at 8 x 2048 rows)
  constexpr int kGLd = kGBK;
  constexpr int BM = 32 * WTM;
  const size_t lds = (size_t)2 * (BM + 128) * kGLd * 2;
  if (!granted) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_tiles_kernel<DT, false, WTM, 4, PF, true, kGBK, 4>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) { set_last_error("%s: cannot reserve %zu bytes of LDS: %s", who, lds, hipGetErrorString(e)); return kErrLaunch; }
    granted = true;
  }
  const int rows = a.B * a.M;
  MfmaArgs g{a.p, 0, 0, a.u, nullptr, a.ldu, a.bias, nullptr, 0, a.y, 0, rows, a.heads * 128, a.R, 0};
  ExpandEpi ep{a.cos, a.sin, a.rope_len, a.positions, a.M, a.sp_b, a.sp_m, a.sy_b, a.sy_m, a.sy_h, a.dst_by_position, a.dst_rows};
  const dim3 grid(a.heads, (rows + BM - 1) / BM);
  hipLaunchKernelGGL((gemm_tiles_kernel<DT, false, WTM, 4, PF, true, kGBK, 4>), grid, dim3(kGT4), lds, st, g, ep);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("%s: launch failed: %s", who, hipGetErrorString(e)); return kErrLaunch; }
  return kOk;
}

template <int DT, int WTM>
static int launch_expand_multi_t(const ExpandArgs* d, int n, hipStream_t st) {
  const char* who = "fsvd_lowrank_expand_heads_multi";
  static bool granted = false;
  constexpr int BM = 32 * WTM;
  const size_t lds = (size_t)2 * (BM + 128) * kGBK * 2;
  if (!granted) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&expand_multi_kernel<DT, WTM>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) { set_last_error("%s: cannot reserve %zu bytes of LDS: %s", who, lds, hipGetErrorString(e)); return kErrLaunch; }
    granted = true;
  }
  const int rows = d[0].B * d[0].M;
  ExpandBatch eb{};
  int heads = 0;
  for (int k = 0; k < 3; ++k) {
    const ExpandArgs& a = d[k < n ? k : n - 1];
    eb.a[k] = MfmaArgs{a.p, 0, 0, a.u, nullptr, a.ldu, a.bias, nullptr, 0, a.y, 0, rows, a.heads * 128, a.R, 0};
    eb.ep[k] = ExpandEpi{a.cos, a.sin, a.rope_len, a.positions, a.M, a.sp_b, a.sp_m, a.sy_b, a.sy_m, a.sy_h, a.dst_by_position, a.dst_rows};
    eb.first_head[k] = heads;
    if (k < n) heads += a.heads;
  }
  eb.first_head[3] = heads;
  for (int k = n; k < 3; ++k) eb.first_head[k] = heads;    // unused sets start past the last head
  const dim3 grid(heads, (rows + BM - 1) / BM);
  hipLaunchKernelGGL((expand_multi_kernel<DT, WTM>), grid, dim3(kGT4), lds, st, eb);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("%s: launch failed: %s", who, hipGetErrorString(e)); return kErrLaunch; }
  return kOk;
}

// the batched form applies when every expansion would take the tiled kernel and they cover the same token rows
bool expand_multi_apply(const ExpandArgs* d, int n) {
  if (n < 2 || n > 3) return false;
  for (int k = 0; k < n; ++k)
    if (!expand_tiles_apply(d[k]) || d[k].B != d[0].B || d[k].M != d[0].M || d[k].dt != d[0].dt) return false;
  return true;
}
int launch_expand_multi(const ExpandArgs* d, int n, hipStream_t st) {
  int heads = 0;
  for (int k = 0; k < n; ++k) heads += d[k].heads;
  const int64_t big = (int64_t)heads * (((int64_t)d[0].B * d[0].M + 127) / 128);
  if (d[0].dt == 1) return big >= 384 ? launch_expand_multi_t<1, 4>(d, n, st) : launch_expand_multi_t<1, 2>(d, n, st);
  return big >= 384 ? launch_expand_multi_t<0, 4>(d, n, st) : launch_expand_multi_t<0, 2>(d, n, st);
}

int launch_expand_tiles(const ExpandArgs& a, hipStream_t st) {
  // a column tile is always one head; 128 token rows per workgroup when that gives every compute unit two tiles, else 64
  const int64_t big = (int64_t)a.heads * (((int64_t)a.B * a.M + 127) / 128);
  if (a.dt == 1) return big >= 384 ? launch_expand_tiles_t<1, 4>(a, st) : launch_expand_tiles_t<1, 2>(a, st);
  return big >= 384 ? launch_expand_tiles_t<0, 4>(a, st) : launch_expand_tiles_t<0, 2>(a, st);
}

}  // namespace fsvd
