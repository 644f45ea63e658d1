// The hand-off of the persistent decode step, alone: every workgroup of a co-resident grid writes its 16 words of a
// tagged vector (tag << 16 | payload, write-through agent-scope stores) and then polls the whole vector with 16-byte
// coherent loads until every tag is the round's, for `rounds` rounds in one launch.  No weights, no arithmetic: what a
// round takes is what a dependent phase of the step costs before it has streamed a byte.  Diagnostic only (bench.py
// prints it next to the step's own figures); the stores, loads and tag scheme are those of decode_step.hip.
#include "common.hpp"
#include "kernels.hpp"

namespace fsvd {

constexpr int kHpThreads = 512;

// both loads of a round and the wait for them are one statement: a load left in flight behind its statement may find
// its destination registers reused before the data lands
__device__ __forceinline__ void hp_poll(u32x4_t (&v)[2], const uint32_t* a0, const uint32_t* a1) {
  asm volatile("global_load_dwordx4 %0, %2, off sc0 sc1\n\tglobal_load_dwordx4 %1, %3, off sc0 sc1\n\ts_waitcnt vmcnt(0)"
               : "=&v"(v[0]), "=&v"(v[1]) : "v"(a0), "v"(a1) : "memory");
}

// vec: [2][16 * gridDim.x] words, zero before the launch; out[0] counts workgroups that gave up after `spin` polls of a round (all others then leave too),
// out[1] the polling rounds that came back stale.  Two buffers in turn: a workgroup can be one round ahead of the
// slowest (it cannot finish round r + 1 before everybody has published it), never two.
__global__ __launch_bounds__(kHpThreads) void handoff_probe_kernel(uint32_t* vec, uint32_t* out, int rounds, int delay, int spin) {
  const int tid = threadIdx.x, wg = blockIdx.x, n = 16 * (int)gridDim.x;
  uint32_t stale = 0, sink = 0;
  for (int r = 1; r <= rounds; ++r) {
    uint32_t* v = vec + (r & 1) * n;
    const uint32_t tag = (uint32_t)r & 0xffffu;
    if (tid < 16) __hip_atomic_store(v + wg * 16 + tid, (tag << 16) | (uint32_t)(wg & 0xffff), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (int d = 0; d < delay; ++d) __builtin_amdgcn_s_sleep(1);   // 64 clocks each: a first poll that leaves at once always comes back stale
    bool fresh = false;
    for (int it = 0; it < spin; ++it) {
      bool mine = true;
      for (int w0 = tid * 8; w0 < n; w0 += kHpThreads * 8) {       // 8 words per lane and trip (n is a multiple of 8)
        u32x4_t x[2];
        hp_poll(x, v + w0, v + w0 + 4);
        mine = mine && (x[0].x >> 16) == tag && (x[0].y >> 16) == tag && (x[0].z >> 16) == tag && (x[0].w >> 16) == tag &&
               (x[1].x >> 16) == tag && (x[1].y >> 16) == tag && (x[1].z >> 16) == tag && (x[1].w >> 16) == tag;
        sink += x[0].x ^ x[1].w;
      }
      if (__syncthreads_and(mine ? 1 : 0)) { fresh = true; break; }
      ++stale;
      // somebody else has given up (a starved grid): leave as well instead of waiting out every round
      if ((it & 255) == 255 && __syncthreads_or(tid == 0 && __hip_atomic_load(out, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)) break;
    }
    if (!fresh) {                                  // uniform over the workgroup: `fresh` comes out of a barrier
      if (tid == 0) atomicAdd(out + 0, 1u);
      break;
    }
  }
  if (tid == 0) {
    atomicAdd(out + 1, stale);
    if (sink == 0x9e3779b9u) out[2] = sink;        // keeps the polled words alive
  }
}

int launch_handoff_probe(uint32_t* vec, uint32_t* out, int workgroups, int rounds, int delay, int spin, hipStream_t st) {
  hipLaunchKernelGGL(handoff_probe_kernel, dim3(workgroups), dim3(kHpThreads), 0, st, vec, out, rounds, delay, spin);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_last_error("fsvd_handoff_probe: launch failed: %s", hipGetErrorString(e)); return kErrLaunch; }
  return kOk;
}

}  // namespace fsvd
