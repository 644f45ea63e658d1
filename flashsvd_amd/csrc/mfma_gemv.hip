// Decode projections for 3..64 rows at once (batched decoding, token-tiled MLP) on the matrix cores.
//
// At batch 1 a projection is a row-dot GEMV on the vector ALU; from a handful of rows on, the vector
// path has to re-read the activations from LDS once per weight row and row of the batch and runs out of
// LDS bandwidth long before HBM is busy.  Here a wave owns 16 weight rows and a slice of K (2, 4 or 8 waves
// share one 16-row tile),
// each wave feeds 16 rows x 32 k of W (A operand) and 16 batch rows x 32 k of X (B operand, read straight
// from L2: the batch is tiny) to V_MFMA_F32_16X16X32_BF16 and accumulates a 16 x 16 fp32 tile per 16
// batch rows; the waves' tiles are added in wave order through LDS (deterministic) and the epilogue
// applies the rounding points of the vector kernels: bias, one bf16 rounding, residual, or SwiGLU.
// Two forms of the weight stream: fragments loaded straight from global memory (16 rows x 64 bytes per instruction;
// any K that is a multiple of 32, up to 64 rows), and, up to 32 rows with K a whole number of 128- / 256-byte pieces,
// whole row pieces loaded into a wave-private LDS ring and fragments read from there (a third faster).
#include "common.hpp"
#include "kernels.hpp"

namespace fsvd {

typedef const __attribute__((address_space(1))) u32x4_t* gp16_t;

constexpr int kMfThreads = 512;
constexpr int kMfWaves = kMfThreads / 64;

template <class F>
__device__ __forceinline__ F ldw_frag(const uint16_t* p) {
  return __builtin_bit_cast(F, __builtin_nontemporal_load((gp16_t)(uintptr_t)p));
}
template <class F>
__device__ __forceinline__ F ldx_frag(const uint16_t* p) {
  return __builtin_bit_cast(F, *(gp16_t)(uintptr_t)p);
}


// the waves' partial tiles through LDS, added in wave order, then the epilogue of the vector kernels
template <int DT, int NB, bool DUAL, int KS>
__device__ __forceinline__ void mfma_finish(const MfmaArgs& a, float (*red)[DUAL ? 2 : 1][NB][4][64], const f32x4_t (&acc)[DUAL ? 2 : 1][NB]) {
  typedef E16<DT> E;
  typedef typename E::frag_t frag_t;
  constexpr int NM = DUAL ? 2 : 1;
  constexpr int RT = kMfWaves / KS;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int t = 0; t < NB; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][m][t][i][lane] = acc[m][t][i];
  __syncthreads();
  // one thread per output element of the RT tiles of 16 x (16 * NB): element i of lane l is row
  // (l / 16) * 4 + i, batch column l % 16; the KS partial tiles are added in wave order
  for (int o = tid; o < RT * NB * 256; o += kMfThreads) {
    const int q = o / (NB * 256), oo = o - q * (NB * 256);
    const int t = oo >> 8, r = oo & 255, i = r >> 6, l = r & 63;
    const int n = (blockIdx.x * RT + q) * 16 + (l >> 4) * 4 + i, b = t * 16 + (l & 15);
    float v0 = 0.f, v1 = 0.f;
#pragma unroll
    for (int w = 0; w < KS; ++w) {
      v0 += red[q * KS + w][0][t][i][l];
      if (DUAL) v1 += red[q * KS + w][NM - 1][t][i][l];
    }
    if (n >= a.N || b >= a.B) continue;
    float v;
    if (DUAL) {
      if (a.mode == 0) {
        v0 = E::rnd(v0);
        v1 = E::rnd(v1);
        v = E::rnd(E::rnd(silu_f32(v0)) * v1);
      } else {
        v = E::rnd((v0 * (1.0f / (1.0f + expf(-v0)))) * v1);
      }
    } else {
      if (a.bias) v0 += E::val(a.bias[n]);
      v = E::rnd(v0);
      if (a.res) v = E::rnd(E::val(a.res[(int64_t)b * a.ldres + n]) + v);
    }
    a.y[(int64_t)b * a.ldy + n] = (uint16_t)E::bits(v);
  }
}

// K split over the gridDim.y workgroups of a weight tile (single matrix): the workgroup's sum of every output element is
// parked in the caller's workspace with write-through agent-scope stores, the arrival is counted once all of them are
// acknowledged, and the last workgroup to arrive adds the gridDim.y shares in split order (its own included, so the sum
// does not depend on who came last) through agent-scope loads, all in flight at once, then applies the epilogue.  No
// fence: a release or acquire fence writes back or empties a whole L2 under the weight streams of the other workgroups.
template <int DT, int NB, int KS>
__device__ __forceinline__ void mfma_finish_split(const MfmaArgs& a, float (*red)[1][NB][4][64], const f32x4_t (&acc)[1][NB]) {
  typedef E16<DT> E;
  typedef typename E::frag_t frag_t;
  constexpr int RT = kMfWaves / KS;
  constexpr int NE = RT * NB * 256;                 // output elements of this workgroup
  constexpr int kMaxZ = 8;
  __shared__ int last_flag;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int Z = gridDim.y;
#pragma unroll
  for (int t = 0; t < NB; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][0][t][i][lane] = acc[0][t][i];
  __syncthreads();
  uint32_t* part = reinterpret_cast<uint32_t*>(a.ws_part) + (size_t)blockIdx.x * Z * NE;
  for (int o = tid; o < NE; o += kMfThreads) {
    const int q = o / (NB * 256), oo = o - q * (NB * 256);
    const int t = oo >> 8, r = oo & 255, i = r >> 6, l = r & 63;
    float v0 = 0.f;
#pragma unroll
    for (int w = 0; w < KS; ++w) v0 += red[q * KS + w][0][t][i][l];
    __hip_atomic_store(part + (size_t)blockIdx.y * NE + o, __float_as_uint(v0), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (tid == 0) {
    const int prev = atomicAdd(a.ws_count + blockIdx.x, 1);
    const int last = prev == Z - 1;
    if (last) a.ws_count[blockIdx.x] = 0;          // ready for the next launch
    last_flag = last;
  }
  __syncthreads();
  if (last_flag == 0) return;
  for (int o = tid; o < NE; o += kMfThreads) {
    const int q = o / (NB * 256), oo = o - q * (NB * 256);
    const int t = oo >> 8, r = oo & 255, i = r >> 6, l = r & 63;
    const int n = (blockIdx.x * RT + q) * 16 + (l >> 4) * 4 + i, b = t * 16 + (l & 15);
    uint32_t sh[kMaxZ];
#pragma unroll
    for (int z = 0; z < kMaxZ; ++z) sh[z] = __hip_atomic_load(part + (size_t)min(z, Z - 1) * NE + o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    float v0 = 0.f;
#pragma unroll
    for (int z = 0; z < kMaxZ; ++z)
      if (z < Z) v0 += __uint_as_float(sh[z]);
    if (n >= a.N || b >= a.B) continue;
    if (a.bias) v0 += E::val(a.bias[n]);
    float v = E::rnd(v0);
    if (a.res) v = E::rnd(E::val(a.res[(int64_t)b * a.ldres + n]) + v);
    a.y[(int64_t)b * a.ldy + n] = (uint16_t)E::bits(v);
  }
}

// NB: 16-row batch tiles (B <= 16 * NB); KS: waves that split K for one 16-row weight tile, so a workgroup
// of 8 waves covers 8 / KS weight tiles
template <int DT, int NB, bool DUAL, int KS>
__global__ __launch_bounds__(kMfThreads) void mfma_linear_kernel(MfmaArgs a) {
  typedef E16<DT> E;
  typedef typename E::frag_t frag_t;
  constexpr int NM = DUAL ? 2 : 1;
  constexpr int RT = kMfWaves / KS;
  __shared__ float red[kMfWaves][NM][NB][4][64];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lr = lane & 15, lg = lane >> 4;
  const int rt = wave / KS, ks = wave % KS;
  const int n0 = (blockIdx.x * RT + rt) * 16;
  const int ksteps = a.K >> 5;
  // the KS waves of a weight tile take the k-steps in turn (wave ks: steps ks, ks + KS, ...), so that together they read
  // KS * 64 contiguous bytes of every row at a time; s counts this wave's own steps
  const int s0 = 0, s1 = (ksteps - ks + KS - 1) / KS;
  const int64_t wo = (int64_t)min(n0 + lr, a.N - 1) * a.ldw + lg * 8;
  const uint16_t* w0 = a.W + wo;
  const uint16_t* w1 = DUAL ? a.W2 + wo : nullptr;
  const uint16_t* xr[NB];
#pragma unroll
  for (int t = 0; t < NB; ++t) xr[t] = a.x + (int64_t)min(t * 16 + lr, a.B - 1) * a.ldx + lg * 8;
  f32x4_t acc[NM][NB];
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int t = 0; t < NB; ++t) acc[m][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  // four k-steps per trip, all loads of a trip requested before the first product; steps past the end of
  // this wave's slice read the last step again and contribute zero
  constexpr int UN = 4;
  const frag_t zero = __builtin_bit_cast(frag_t, u32x4_t{0u, 0u, 0u, 0u});
  for (int s = s0; s < s1; s += UN) {
    frag_t fa0[UN], fa1[UN], fb0[UN][NB], fb1[UN][NB];
#pragma unroll
    for (int j = 0; j < UN; ++j) {
      const int k = (min(s + j, s1 - 1) * KS + ks) << 5;
      fa0[j] = ldw_frag<frag_t>(w0 + k);
      if (DUAL) fa1[j] = ldw_frag<frag_t>(w1 + k);
#pragma unroll
      for (int t = 0; t < NB; ++t) {
        fb0[j][t] = ldx_frag<frag_t>(xr[t] + k);
        if (DUAL) fb1[j][t] = ldx_frag<frag_t>(xr[t] + a.up_off + k);
      }
    }
#pragma unroll
    for (int j = 0; j < UN; ++j) {
      const bool live = s + j < s1;
      const frag_t a0 = live ? fa0[j] : zero;
#pragma unroll
      for (int t = 0; t < NB; ++t) {
        acc[0][t] = E::mfma(a0, fb0[j][t], acc[0][t]);
        if (DUAL) acc[1][t] = E::mfma(live ? fa1[j] : zero, fb1[j][t], acc[1][t]);
      }
    }
  }
  mfma_finish<DT, NB, DUAL, KS>(a, red, acc);
}

// ---------------------------------------------------------------------------------------------
// Up to 16 rows: the same decomposition (a wave = 16 weight rows x a share of K, partial tiles added in wave order), but
// the weights arrive the way the batch-1 kernels read them: whole 128- or 256-byte pieces of a row, loaded straight into
// a ring of LDS stages that belongs to the wave (no barrier in the loop, only the wave's own load counter), and the
// matrix-core fragments are read from there.  The fragment loads of the kernel above touch 16 rows x 64 bytes per
// instruction; timing that kernel with 1 KB-contiguous loads of the same volume (wrong results, same traffic) showed the
// access pattern to cost a third of its time.  LDS position p of a row holds piece p ^ (row % pieces): conflict-free
// 16-byte fragment reads (see mfma_gemm.hip).
// ---------------------------------------------------------------------------------------------
template <bool DUAL> struct StreamShape {
  static constexpr int CKB = DUAL ? 128 : 256;     // bytes of a weight row per chunk
  static constexpr int NM = DUAL ? 2 : 1;
  static constexpr int kStage = NM * 16 * CKB;     // 4 KB either way
};

// D: chunks in a wave's ring (D - 1 in flight while one multiplies)
// ZS: K also split over the gridDim.y workgroups of a tile (single matrix; narrow projections that would otherwise
// leave compute units idle): the KS waves of workgroup z act as waves z * KS .. z * KS + KS - 1 of KS * gridDim.y
template <int DT, bool DUAL, int KS, int D, int NB, bool ZS = false>
__global__ __launch_bounds__(kMfThreads) void mfma_stream_kernel(MfmaArgs a) {
  typedef E16<DT> E;
  typedef typename E::frag_t frag_t;
  static_assert(!ZS || !DUAL, "the split over workgroups is built for a single matrix");
  typedef StreamShape<DUAL> SS;
  constexpr int NM = SS::NM, CKB = SS::CKB, kStage = SS::kStage;
  constexpr int RT = kMfWaves / KS;
  constexpr int PPR = CKB / 16;                    // 16-byte pieces per row and chunk
  constexpr int KST = CKB / 64;                    // k-steps of 32 per chunk
  constexpr int RPI = 64 / PPR;                    // rows one load instruction covers (64 lanes x 16 bytes)
  constexpr int NI = 16 / RPI;                     // load instructions per matrix and chunk
  constexpr int kGroup = NM * NI + NM * KST * NB;  // loads per chunk: weight pieces into LDS, activation fragments into registers
  static_assert((D - 1) * kGroup < 64 && D >= 2 && D <= 4, "vmcnt holds six bits; the waits below cover up to three groups in flight");
  extern __shared__ __align__(16) unsigned char st_smem[];     // [8 waves][D][kStage]; the partial tiles at the end
  float (*red)[NM][NB][4][64] = reinterpret_cast<float (*)[NM][NB][4][64]>(st_smem);
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lr = lane & 15, lg = lane >> 4;
  const int rt = wave / KS, ks = ZS ? (int)blockIdx.y * KS + wave % KS : wave % KS;
  const int KSV = ZS ? KS * (int)gridDim.y : KS;   // waves that share a weight tile
  const int n0 = (blockIdx.x * RT + rt) * 16;
  unsigned char* ring = st_smem + (size_t)wave * D * kStage;
  const int nchunk = a.K / (CKB / 2);
  const int cw = max(0, (nchunk - ks + KSV - 1) / KSV);   // this wave's chunks: ks, ks + KSV, ... (the waves of a tile read adjacent pieces)
  typedef const __attribute__((address_space(1))) void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;
  const int lrow = lane / PPR, lpc = lane % PPR;
  const uint16_t* wsrc[NM][NI];
#pragma unroll
  for (int q = 0; q < NI; ++q) {
    const int row = q * RPI + lrow;
    const int64_t off = (int64_t)min(n0 + row, a.N - 1) * a.ldw + ((lpc ^ (row % PPR)) * 8);
    wsrc[0][q] = a.W + off;
    if (DUAL) wsrc[NM - 1][q] = a.W2 + off;
  }
  const uint16_t* xsrc[NB];
#pragma unroll
  for (int t = 0; t < NB; ++t) xsrc[t] = a.x + (int64_t)min(t * 16 + lr, a.B - 1) * a.ldx + lg * 8;
  frag_t xf[D][NM][KST][NB];
  // The wave's load counter is the only synchronisation: it counts weight pieces and activation fragments alike, in
  // issue order, so the loads of one chunk must stay together in the instruction stream (scheduling fences around them).
  const auto issue = [&](int c, int slot) {
    const int k0 = (c * KSV + ks) * (CKB / 2);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < NM; ++m) {
#pragma unroll
      for (int q = 0; q < NI; ++q)
        __builtin_amdgcn_global_load_lds((gptr_t)(wsrc[m][q] + k0), (lptr_t)(ring + slot * kStage + m * 16 * CKB + q * 1024), 16, 0, 2);
#pragma unroll
      for (int s = 0; s < KST; ++s)
#pragma unroll
        for (int t = 0; t < NB; ++t) xf[slot][m][s][t] = ldx_frag<frag_t>(xsrc[t] + (m ? a.up_off : 0) + k0 + s * 32);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  f32x4_t acc[NM][NB];
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int t = 0; t < NB; ++t) acc[m][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  // load counter values that leave the newest r groups in flight
  constexpr int kW0 = (7 << 4) | (15 << 8);
  const auto vm = [](int n) { return (n & 15) | ((n >> 4) << 14); };
#pragma unroll
  for (int c = 0; c < D - 1; ++c)
    if (c < cw) issue(c, c);
  for (int c0 = 0; c0 < cw; c0 += D) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      const int c = c0 + u;
      if (c >= cw) break;
      if (c + D - 1 < cw) issue(c + D - 1, (u + D - 1) % D);
      // chunk c has landed once no more than the groups issued after it are outstanding
      const int newer = min(D - 1, cw - 1 - c);
      if (newer >= 3) __builtin_amdgcn_s_waitcnt(kW0 | vm(3 * kGroup));
      else if (newer == 2) __builtin_amdgcn_s_waitcnt(kW0 | vm(2 * kGroup));
      else if (newer == 1) __builtin_amdgcn_s_waitcnt(kW0 | vm(kGroup));
      else __builtin_amdgcn_s_waitcnt(kW0 | vm(0));
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < KST; ++s)
#pragma unroll
        for (int m = 0; m < NM; ++m) {
          const frag_t wf = *reinterpret_cast<const frag_t*>(ring + u * kStage + m * 16 * CKB + lr * CKB + (((s * 4 + lg) ^ (lr % PPR)) * 16));
#pragma unroll
          for (int t = 0; t < NB; ++t) acc[m][t] = E::mfma(wf, xf[u][m][s][t], acc[m][t]);
        }
    }
  }
  __syncthreads();                                 // every wave is done with its ring: the partial tiles take its place
  if constexpr (ZS) mfma_finish_split<DT, NB, KS>(a, red, acc);
  else mfma_finish<DT, NB, DUAL, KS>(a, red, acc);
}

// ---------------------------------------------------------------------------------------------
// Wide matrices (at least two 16-row tiles per compute unit) at up to 32 rows: the same wave-private LDS ring, but one
// workgroup per compute unit that stays for the whole matrix.  Workgroup g takes tiles g, g + G, g + 2G, ...; its eight
// waves split K as above, and because a wave's share of K is the same for every tile, its activation fragments are loaded
// ONCE into registers (CW chunks x KST steps x NB batch tiles).  The loop then holds nothing but weight pieces on their way
// into LDS: the ring runs on across tile boundaries (the pieces of the next tile are in flight while this tile's partial
// sums are added through LDS and stored), and the load counter counts only them.  In the kernel above the activation
// fragments travel with every chunk, and the compiler, which cannot follow register loads around the loop, waits for all
// outstanding loads — the chunk requested ahead included — before every second product.
// ---------------------------------------------------------------------------------------------
constexpr int kResPitch = 68;                      // floats between the four row groups of a parked tile: conflict-free reads below
template <int DT, bool DUAL, int NB, int CW, int D>
__global__ __launch_bounds__(kMfThreads) void mfma_resident_kernel(MfmaArgs a) {
  typedef E16<DT> E;
  typedef typename E::frag_t frag_t;
  typedef StreamShape<DUAL> SS;
  constexpr int NM = SS::NM, CKB = SS::CKB, kStage = SS::kStage;
  constexpr int PPR = CKB / 16, KST = CKB / 64, RPI = 64 / PPR, NI = 16 / RPI;
  constexpr int kGroup = NM * NI;                  // loads per chunk
  constexpr int NE = NB * 256;                      // output elements of a tile
  static_assert(D >= 2 && D <= 4 && 3 * kGroup < 64, "the waits below cover up to three groups in flight");
  extern __shared__ __align__(16) unsigned char st_smem[];     // [8 waves][D][kStage], then the parked partial tiles
  constexpr int kRedWave = NM * NB * 4 * kResPitch;
  float* red = reinterpret_cast<float*>(st_smem + (size_t)kMfWaves * D * kStage);   // [8][NM][NB][4][kResPitch]
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lr = lane & 15, lg = lane >> 4;
  const int tiles = (a.N + 15) / 16, G = gridDim.x, g = blockIdx.x;
  const int nt = (tiles - g + G - 1) / G;          // this workgroup's tiles: g, g + G, ...
  const int nchunk = a.K / (CKB / 2);
  const int cw = min(CW, max(0, (nchunk - wave + kMfWaves - 1) / kMfWaves));   // this wave's chunks: wave, wave + 8, ...
  unsigned char* ring = st_smem + (size_t)wave * D * kStage;
  typedef const __attribute__((address_space(1))) void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;
  const int lrow = lane / PPR, lpc = lane % PPR;

  const int total = nt * cw;
  int issued = 0, it = 0, ic = 0, islot = 0;
  const auto issue = [&]() {
    const int n0 = (g + it * G) * 16;
    const int k0 = (ic * kMfWaves + wave) * (CKB / 2);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
      for (int q = 0; q < NI; ++q) {
        const int row = q * RPI + lrow;
        const uint16_t* src = (m ? a.W2 : a.W) + (int64_t)min(n0 + row, a.N - 1) * a.ldw + ((lpc ^ (row % PPR)) * 8) + k0;
        __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(ring + islot * kStage + m * 16 * CKB + q * 1024), 16, 0, 2);
      }
    __builtin_amdgcn_sched_barrier(0);
    ++issued;
    if (++ic == cw) { ic = 0; ++it; }
    islot = islot + 1 == D ? 0 : islot + 1;
  };
  constexpr int kW0 = (7 << 4) | (15 << 8);
  const auto vm = [](int n) { return (n & 15) | ((n >> 4) << 14); };
#pragma unroll
  for (int p = 0; p < D; ++p)
    if (issued < total) issue();
  // the wave's activation fragments, requested behind the first weight stages so that both are on their way together
  frag_t xf[CW][NM][KST][NB];
  const frag_t zero = __builtin_bit_cast(frag_t, u32x4_t{0u, 0u, 0u, 0u});
#pragma unroll
  for (int c = 0; c < CW; ++c)
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
      for (int s = 0; s < KST; ++s)
#pragma unroll
        for (int t = 0; t < NB; ++t)
          xf[c][m][s][t] = c < cw ? ldx_frag<frag_t>(a.x + (int64_t)min(t * 16 + lr, a.B - 1) * a.ldx + lg * 8 + (m ? a.up_off : 0) +
                                             (int64_t)(c * kMfWaves + wave) * (CKB / 2) + s * 32)
                                  : zero;
  __builtin_amdgcn_s_waitcnt(0);                   // (the first stages land with them) from here on the load counter counts weight pieces only
  __builtin_amdgcn_sched_barrier(0);

  int done = 0, cslot = 0;
  // one thread per output element, 16 consecutive lanes on 16 consecutive columns of one batch row (32-byte stores):
  // element i of lane l of a tile is weight row (l / 16) * 4 + i, batch row l % 16
  const int nn = tid & 15, b = tid >> 4;
  const int ro = ((b >> 4) * 4 + (nn & 3)) * kResPitch + (nn >> 2) * 16 + (b & 15);
  for (int ti = 0; ti < nt; ++ti) {
    f32x4_t acc[NM][NB];
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
      for (int t = 0; t < NB; ++t) acc[m][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < CW; ++c) {
      if (c < cw) {
        // chunk `done` has landed once no more than the groups requested after it are outstanding (stores of the
        // epilogue below, where they sit between two groups, only make this wait a little stricter)
        const int newer = issued - done - 1;
        if (newer >= 3) __builtin_amdgcn_s_waitcnt(kW0 | vm(3 * kGroup));
        else if (newer == 2) __builtin_amdgcn_s_waitcnt(kW0 | vm(2 * kGroup));
        else if (newer == 1) __builtin_amdgcn_s_waitcnt(kW0 | vm(kGroup));
        else __builtin_amdgcn_s_waitcnt(kW0 | vm(0));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < KST; ++s)
#pragma unroll
          for (int m = 0; m < NM; ++m) {
            const frag_t wf = *reinterpret_cast<const frag_t*>(ring + cslot * kStage + m * 16 * CKB + lr * CKB + (((s * 4 + lg) ^ (lr % PPR)) * 16));
#pragma unroll
            for (int t = 0; t < NB; ++t) acc[m][t] = E::mfma(wf, xf[c][m][s][t], acc[m][t]);
          }
        ++done;
        cslot = cslot + 1 == D ? 0 : cslot + 1;
        // the stage is free again (its fragments are in registers): the chunk D ahead goes into it at once, so that a
        // tile's last stages are on their way again before the partial sums are added
        if (issued < total) issue();
      }
    }
    // the waves' partial tiles through LDS, added in wave order; bare barrier instructions: __syncthreads() carries a
    // fence that waits for all of the wave's loads, the pieces requested ahead included
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
      for (int t = 0; t < NB; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[wave * kRedWave + ((m * NB + t) * 4 + i) * kResPitch + lane] = acc[m][t][i];
    __builtin_amdgcn_s_waitcnt(0xc07f);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    const int n = (g + ti * G) * 16 + nn;
    if (tid < NE) {
      float v0 = 0.f, v1 = 0.f;
#pragma unroll
      for (int w = 0; w < kMfWaves; ++w) {
        v0 += red[w * kRedWave + ro];
        if (DUAL) v1 += red[w * kRedWave + (NM - 1) * NB * 4 * kResPitch + ro];
      }
      if (n < a.N && b < a.B) {
        float v;
        if (DUAL) {
          if (a.mode == 0) {
            v0 = E::rnd(v0);
            v1 = E::rnd(v1);
            v = E::rnd(E::rnd(silu_f32(v0)) * v1);
          } else {
            v = E::rnd((v0 * (1.0f / (1.0f + expf(-v0)))) * v1);
          }
        } else {
          if (a.bias) v0 += E::val(a.bias[n]);
          v = E::rnd(v0);
          if (a.res) v = E::rnd(E::val(a.res[(int64_t)b * a.ldres + n]) + v);
        }
        a.y[(int64_t)b * a.ldy + n] = (uint16_t)E::bits(v);
      }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);            // the sums are in registers before the next tile's partials overwrite them
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  }
}

static int compute_units() {
  static int cus[16] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return 0;
  if (cus[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    cus[dev] = n;
  }
  return cus[dev];
}
// The resident form applies to 8..32 rows of a matrix with at least two tiles per compute unit whose K is a whole number
// of chunks, one to six per wave.  Measured against the one-shot kernels at the 7B shapes (us per call at 8 / 16 / 32
// rows): gate/up pair 14.5 -> 13.6 / 17.5 -> 14.9 / 24.7 -> 18.7, q|k|v expansion 8.1 -> 8.1 / 9.3 -> 8.5 / 11.2 -> 10.0,
// lm_head 45.2 -> 45.3 / 54.9 -> 46.7 / 78.1 -> 53.4; at 3 rows it is 3-5 % behind, and narrower matrices (one tile per
// workgroup, with or without K split over workgroups as well) are where they were or slower, so both stay where they are.
constexpr int kResidentCW = 6;
template <bool DUAL>
static bool resident_applies(const MfmaArgs& a) {
  constexpr int ck = StreamShape<DUAL>::CKB / 2;
  const int cu = compute_units();
  if (cu <= 0 || a.B < 8 || a.B > 32 || (a.K % ck) != 0) return false;
  const int nchunk = a.K / ck;
  return (a.N + 15) / 16 >= 2 * cu && nchunk >= kMfWaves && nchunk <= kMfWaves * kResidentCW;
}
template <int DT, bool DUAL, int NB, int CW>
static int launch_mfma_resident_t(const MfmaArgs& a, hipStream_t st, const char* who) {
  static bool granted = false;
  constexpr int D = 3;
  constexpr int NM = StreamShape<DUAL>::NM;
  const size_t lds = (size_t)kMfWaves * D * StreamShape<DUAL>::kStage + (size_t)kMfWaves * NM * NB * 4 * kResPitch * sizeof(float);
  const void* f = reinterpret_cast<const void*>(&mfma_resident_kernel<DT, DUAL, NB, CW, D>);
  if (!granted) {
    hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) { set_last_error("%s: cannot reserve %zu bytes of LDS: %s", who, lds, hipGetErrorString(e)); return kErrLaunch; }
    granted = true;
  }
  const int G = std::min(compute_units(), (a.N + 15) / 16);
  hipLaunchKernelGGL((mfma_resident_kernel<DT, DUAL, NB, CW, D>), dim3(G), dim3(kMfThreads), lds, st, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("%s: launch failed: %s", who, hipGetErrorString(e)); return kErrLaunch; }
  return kOk;
}
template <int DT, bool DUAL, int NB>
static int launch_mfma_resident_nb(const MfmaArgs& a, hipStream_t st, const char* who) {
  const int per = (a.K / (StreamShape<DUAL>::CKB / 2) + kMfWaves - 1) / kMfWaves;   // chunks of the busiest wave
  if (per <= 2) return launch_mfma_resident_t<DT, DUAL, NB, 2>(a, st, who);
  if (per <= 4) return launch_mfma_resident_t<DT, DUAL, NB, 4>(a, st, who);
  return launch_mfma_resident_t<DT, DUAL, NB, 6>(a, st, who);
}
template <int DT, bool DUAL>
static int launch_mfma_resident(const MfmaArgs& a, hipStream_t st, const char* who) {
  return a.B <= 16 ? launch_mfma_resident_nb<DT, DUAL, 1>(a, st, who) : launch_mfma_resident_nb<DT, DUAL, 2>(a, st, who);
}

template <int DT, int NB, bool DUAL>
static void launch_mfma_ks(const MfmaArgs& a, int ks, hipStream_t st) {
  const int tiles = (a.N + 15) / 16;
  const dim3 block(kMfThreads);
  if (ks == 2) hipLaunchKernelGGL((mfma_linear_kernel<DT, NB, DUAL, 2>), dim3((tiles + 3) / 4), block, 0, st, a);
  else if (ks == 4) hipLaunchKernelGGL((mfma_linear_kernel<DT, NB, DUAL, 4>), dim3((tiles + 1) / 2), block, 0, st, a);
  else hipLaunchKernelGGL((mfma_linear_kernel<DT, NB, DUAL, 8>), dim3(tiles), block, 0, st, a);
}

// the streaming form: up to 16 rows, K a whole number of chunks with at least one chunk per wave of a tile
template <bool DUAL>
static bool stream_applies(const MfmaArgs& a, int ks) {
  constexpr int ck = StreamShape<DUAL>::CKB / 2;
  return a.B <= 32 && (a.K % ck) == 0 && a.K / ck >= ks;
}
template <int DT, bool DUAL, int D, int NB>
static int launch_mfma_stream_d(const MfmaArgs& a, int ks, hipStream_t st, const char* who) {
  static bool granted[3] = {false, false, false};
  const int tiles = (a.N + 15) / 16;
  const size_t lds = (size_t)kMfWaves * D * StreamShape<DUAL>::kStage;
  const auto grant = [&](const void* f, int i) {
    if (granted[i] || lds <= 64 * 1024) return true;
    hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) { set_last_error("%s: cannot reserve %zu bytes of LDS: %s", who, lds, hipGetErrorString(e)); return false; }
    return granted[i] = true;
  };
  const dim3 block(kMfThreads);
  if (ks == 2) {
    if (!grant(reinterpret_cast<const void*>(&mfma_stream_kernel<DT, DUAL, 2, D, NB>), 0)) return kErrLaunch;
    hipLaunchKernelGGL((mfma_stream_kernel<DT, DUAL, 2, D, NB>), dim3((tiles + 3) / 4), block, lds, st, a);
  } else if (ks == 4) {
    if (!grant(reinterpret_cast<const void*>(&mfma_stream_kernel<DT, DUAL, 4, D, NB>), 1)) return kErrLaunch;
    hipLaunchKernelGGL((mfma_stream_kernel<DT, DUAL, 4, D, NB>), dim3((tiles + 1) / 2), block, lds, st, a);
  } else {
    if (!grant(reinterpret_cast<const void*>(&mfma_stream_kernel<DT, DUAL, 8, D, NB>), 2)) return kErrLaunch;
    hipLaunchKernelGGL((mfma_stream_kernel<DT, DUAL, 8, D, NB>), dim3(tiles), block, lds, st, a);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("%s: launch failed: %s", who, hipGetErrorString(e)); return kErrLaunch; }
  return kOk;
}
// Eight waves per weight tile whenever K has a chunk for each, and a ring of two chunks: 64 KB of LDS, so two
// workgroups share a compute unit — measured better than deeper rings with one workgroup per compute unit or fewer waves
// per tile (7B MLP at 8 rows, ring 4 / 2: rank projection 8.9 / 7.9 us, pair 19.7 / 15.9, down_u 4.9 / 4.9).
template <int DT, bool DUAL>
static int launch_mfma_stream(const MfmaArgs& a, int ks, hipStream_t st, const char* who) {
  if (a.K / (StreamShape<DUAL>::CKB / 2) >= 8) ks = 8;
  return a.B <= 16 ? launch_mfma_stream_d<DT, DUAL, 2, 1>(a, ks, st, who) : launch_mfma_stream_d<DT, DUAL, 2, 2>(a, ks, st, who);
}

// Narrow projections (fewer than 128 weight tiles, e.g. down_v of the 7B MLP: 96) at 3..32 rows: the streaming form with
// K split over up to eight workgroups per tile as well, enough to give every compute unit about two workgroups while
// every wave keeps at least one chunk.  Needs the registered workspace.  Measured per call, 32-row tiles split over
// workgroups -> this form: down_v (1536 x 11008, five shares) 16.4 -> 12.2 us at 8 rows, 17.4 -> 16.6 at 32 rows; o_v
// (1024 x 4096, four shares) 8.7 -> 6.2 at 8 rows, 8.8 -> 7.5 at 32 rows.
constexpr int kStreamSplitMax = 8;
static int stream_split_shares(const MfmaArgs& a) {
  constexpr int ck = StreamShape<false>::CKB / 2;
  if (a.B > 32 || (a.K % ck) != 0) return 1;
  const SplitWorkspace ws = split_workspace();
  const int tiles = (a.N + 15) / 16, nchunk = a.K / ck;
  if (ws.part == nullptr || tiles > ws.ncount || tiles >= 128) return 1;
  const size_t share = (size_t)(a.B <= 16 ? 1 : 2) * 256;
  int z = std::min(kStreamSplitMax, (480 + tiles - 1) / tiles);
  while (z > 1 && (nchunk < kMfWaves * z || (size_t)tiles * z * share > ws.part_floats)) --z;
  return z;
}
template <int DT, int NB>
static int launch_mfma_stream_split(const MfmaArgs& a0, int z, hipStream_t st, const char* who) {
  static bool granted = false;
  constexpr int D = 2;
  const size_t lds = (size_t)kMfWaves * D * StreamShape<false>::kStage;
  const void* f = reinterpret_cast<const void*>(&mfma_stream_kernel<DT, false, 8, D, NB, true>);
  if (!granted && lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) { set_last_error("%s: cannot reserve %zu bytes of LDS: %s", who, lds, hipGetErrorString(e)); return kErrLaunch; }
    granted = true;
  }
  MfmaArgs a = a0;
  const SplitWorkspace ws = split_workspace();
  a.ksplit = z;
  a.ws_part = ws.part;
  a.ws_count = ws.count;
  hipLaunchKernelGGL((mfma_stream_kernel<DT, false, 8, D, NB, true>), dim3((a.N + 15) / 16, z), dim3(kMfThreads), lds, st, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("%s: launch failed: %s", who, hipGetErrorString(e)); return kErrLaunch; }
  return kOk;
}

template <int DT, bool DUAL>
static int launch_mfma(const MfmaArgs& a0, hipStream_t st, const char* who) {
  // K is split over as few waves as still give every compute unit a workgroup: long slices amortise the
  // reduction, but a small matrix needs all eight waves of a workgroup on one weight tile to fill the chip
  const int tiles = (a0.N + 15) / 16, ksteps = a0.K >> 5;
  int ks = 8;
  for (int c = 2; c <= 8; c *= 2)
    if ((tiles * c + 7) / 8 >= 256 && ksteps / c >= 4) { ks = c; break; }
  // many rows (prefill): the tiled kernel reads every weight once per 128 rows instead of once per 64
  if (gemm_tiles_apply(a0)) return launch_gemm_tiles(a0, DUAL, st, who);
  // a batch of rows: 32-row tiles with K split over workgroups, when the caller has registered a workspace — from 33
  // rows on (up to 32 rows the streaming form is faster: 12.3 / 25.3 / 6.7 us against 13.4 / 28.8 / 8.8 us on the wide
  // matrices of the 7B MLP; matrices with fewer than 128 weight tiles take its split form above, or the 32-row tiles
  // when their K does not divide into chunks)
  if (resident_applies<DUAL>(a0)) return launch_mfma_resident<DT, DUAL>(a0, st, who);
  const bool streamed = a0.B <= 32 && tiles >= 128 && stream_applies<DUAL>(a0, ks);
  if constexpr (!DUAL) {
    const int z = stream_split_shares(a0);
    if (z > 1) return a0.B <= 16 ? launch_mfma_stream_split<DT, 1>(a0, z, st, who) : launch_mfma_stream_split<DT, 2>(a0, z, st, who);
  }
  if (gemm_rows_apply(a0) && !streamed) return launch_gemm_rows(a0, DUAL, st, who);
  // batches above 64 rows go in slices of 64
  for (int b0 = 0; b0 < a0.B; b0 += 64) {
    MfmaArgs a = a0;
    a.B = min(64, a0.B - b0);
    a.x = a0.x + (int64_t)b0 * a0.ldx;
    a.y = a0.y + (int64_t)b0 * a0.ldy;
    if (a0.res) a.res = a0.res + (int64_t)b0 * a0.ldres;
    const int nb = (a.B + 15) / 16;
    if (nb <= 2 && stream_applies<DUAL>(a, ks)) {
      const int rc = launch_mfma_stream<DT, DUAL>(a, ks, st, who);
      if (rc != kOk) return rc;
      continue;
    }
    if (nb == 1) launch_mfma_ks<DT, 1, DUAL>(a, ks, st);
    else if (nb == 2) launch_mfma_ks<DT, 2, DUAL>(a, ks, st);
    else if (nb == 3) launch_mfma_ks<DT, 3, DUAL>(a, ks, st);
    else launch_mfma_ks<DT, 4, DUAL>(a, ks, st);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_last_error("%s: launch failed: %s", who, hipGetErrorString(e)); return kErrLaunch; }
  }
  return kOk;
}

static inline bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// true when the matrix-core path applies (the caller then skips the vector kernel)
bool mfma_linear_applies(const LinearArgs& a) {
  return a.B >= 3 && a.norm_w == nullptr && (a.K % 32) == 0 && (a.ldw % 8) == 0 && (a.ldx % 8) == 0 && al16(a.W) && al16(a.x);
}
int launch_linear_mfma(const LinearArgs& a, hipStream_t st) {
  MfmaArgs m{a.x, a.ldx, 0, a.W, nullptr, a.ldw, a.bias, a.res, a.ldres, a.y, a.ldy, a.B, a.N, a.K, 0};
  m.dt = a.dt;
  return a.dt == 1 ? launch_mfma<1, false>(m, st, "fsvd_linear") : launch_mfma<0, false>(m, st, "fsvd_linear");
}
bool mfma_swiglu_applies(const SwigluArgs& a) {
  return a.B >= 3 && (a.R % 32) == 0 && (a.ldw % 8) == 0 && (a.ldp % 8) == 0 && (a.up_off % 8) == 0 && al16(a.gate_u) &&
         al16(a.up_u) && al16(a.p);
}
int launch_swiglu_mfma(const SwigluArgs& a, hipStream_t st) {
  MfmaArgs m{a.p, a.ldp, a.up_off, a.gate_u, a.up_u, a.ldw, nullptr, nullptr, 0, a.h, a.ldh, a.B, a.D, a.R, a.mode};
  m.dt = a.dt;
  return a.dt == 1 ? launch_mfma<1, true>(m, st, "fsvd_swiglu_linear") : launch_mfma<0, true>(m, st, "fsvd_swiglu_linear");
}

}  // namespace fsvd
