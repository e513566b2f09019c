// Sparse down projection over neuron-major weights: y[b,:] = sum over active j of z[b,j] * wdown_t[j,:].
//
// Work split.  Columns are cut into slabs of 64 lanes x 16 bytes (512 fp16 columns = 1 KiB of a row), the
// neurons into `ngroup` equal index ranges.  Workgroup (slab, group) streams the 1 KiB slab segment of every
// active row in its range: the waves deal the active rows round-robin and keep up to U loads in flight per
// lane.  Partial sums stay in registers (VEC per lane per batch row) and are folded across the waves of the
// workgroup through LDS.  Across workgroups there are two ways out:
//   * y_out (dtype output): every workgroup stores its slab partial to scratch, the last workgroup of the slab
//     to finish adds the ngroup partials in group order and writes the rounded result.  No atomics on data
//     (32 workgroups adding into the same 16 cache lines serialise for microseconds), a fixed summation order
//     (bitwise reproducible output), nothing to zero between calls.
//   * y32 (caller's fp32 accumulator, "atomic_gemv" semantics): one fp32 atomic per column per workgroup.
// blockIdx % nslab picks the slab, so with 8 slabs every XCD (workgroups are dealt round-robin over the 8
// XCDs) streams one slab.
//
// The active list is not read from memory: a workgroup turns the mask bytes of its own range into an index
// list in LDS (popcount, wave prefix sum, bit expansion) while the other waves stage the matching z values.
// Both loads are independent, so the prologue costs one memory round trip.  Equal index ranges rather than
// equal shares of the active list: the shares differ by the binomial spread of the active count (a few
// percent at these sizes), which is cheaper than the extra dependent pass a global prefix sum would need.
#pragma once
#include "cats_device.h"

namespace cats {

struct DownArgs {
  const u32x4* wd;        // (I, H) neuron-major
  const void* z;          // (nb, I) fp32 or dtype
  const uint8_t* mask;    // ceil(I/8) bytes, bit j = neuron j active for some batch row
  float* y32;             // (nb, H) the caller's fp32 accumulator (atomics), used when y_out == NULL
  void* y_out;            // (nb, H) dtype
  float* partial;         // y_out mode: [nslab][ngroup][B][64*VEC] fp32 slab partials
  uint32_t* done;         // y_out mode: per-slab arrival counters, zero between calls
  int32_t* count_out;     // optional: number of active neurons
  int H, I, nb;
  int row_vecs;           // H / VEC
  int nslab, ngroup;
  int chunk;              // neurons per group, a multiple of 8
#ifdef CATS_TIMING
  long long* tbuf;        // [gridDim][8] wall-clock stamps (100 MHz) at phase boundaries, development builds only
#endif
};

#ifdef CATS_TIMING
#define CATS_STAMP(slot) do { if (p.tbuf && threadIdx.x == 0) p.tbuf[(size_t)blockIdx.x * 8 + (slot)] = wall_clock64(); } while (0)
#else
#define CATS_STAMP(slot) do { } while (0)
#endif

template <class DT, int B, bool ZF32, int U>
__global__ __launch_bounds__(1024) void down_kernel(DownArgs p) {
  typedef typename DT::st st;
  constexpr int VEC = DT::VEC;
  constexpr int kSlabCols = kWave * VEC;
  extern __shared__ float s_dyn[];
  // dynamic LDS: [chunk] int list | [B][chunk] float z (indexed by j - j0) | [nwaves][64*VEC] float partials
  int* s_list = (int*)s_dyn;
  float* s_z = s_dyn + p.chunk;
  float* s_red = s_z + (size_t)B * p.chunk;
  __shared__ int s_n;
  __shared__ int s_last;

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform by construction; say so
  const int nwaves = blockDim.x >> 6;
  const int slab = blockIdx.x % p.nslab;
  const int group = blockIdx.x / p.nslab;
  const int j0 = group * p.chunk;
  const int j1 = min(j0 + p.chunk, p.I);
  CATS_STAMP(0);

  // ---- 1. wave 0: mask bytes of the range -> ascending index list; the other waves: z of the range -> LDS ----
  if (wave == 0) {
    int base = 0;
    for (int byte0 = j0 >> 3; byte0 * 8 < j1; byte0 += kWave) {
      const int byte = byte0 + lane;
      uint32_t bits = 0;
      if (byte * 8 < j1) {
        bits = p.mask[byte];
        const int rem = j1 - byte * 8;
        if (rem < 8) bits &= (1u << rem) - 1u;
      }
      const int pc = __popc(bits);
      int rank = base + wave_scan_inclusive(pc, lane) - pc;
      while (bits) {
        const int bit = __builtin_ctz(bits);
        bits &= bits - 1;
        s_list[rank++] = byte * 8 + bit;
      }
      base = __shfl(rank, kWave - 1, kWave);  // lane 63 ends at base + (set bits of this pass)
    }
    if (lane == 0) s_n = base;
  } else {
    const int span = j1 - j0;
    for (int b = 0; b < B; b++) {
      for (int q = tid - kWave; q < span; q += blockDim.x - kWave) {
        float zv = 0.f;
        if (b < p.nb) {
          const size_t o = (size_t)b * p.I + j0 + q;
          zv = ZF32 ? ((const float*)p.z)[o] : DT::tof(((const st*)p.z)[o]);
        }
        s_z[b * p.chunk + q] = zv;
      }
    }
  }
  __syncthreads();
  const int n = s_n;
  CATS_STAMP(1);

  // ---- 2. stream the slab segments of the active rows ---------------------------------------------------
  float acc[B][VEC];
#pragma unroll
  for (int b = 0; b < B; b++)
#pragma unroll
    for (int e = 0; e < VEC; e++) acc[b][e] = 0.f;

  // Lanes past the end of a row (H not a multiple of 64 * VEC) re-read the row's last vector; their sums
  // are dropped at the column check below, so no load is predicated per lane.
  const int v = min(slab * kWave + lane, p.row_vecs - 1);
  // This wave owns list entries wave, wave + nwaves, ...; split them into passes of at most U, evenly.
  const int mine = n > wave ? (n - wave + nwaves - 1) / nwaves : 0;
  const int passes = (mine + U - 1) / U;
  const int per = passes ? (mine + passes - 1) / passes : 0;
  for (int t0 = 0; t0 < mine; t0 += per) {
    const int cnt = min(per, mine - t0);  // wave-uniform
    u32x4 wv[U];
    int jj[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      if (u < cnt) {
        jj[u] = s_list[wave + (t0 + u) * nwaves];
        wv[u] = load_stream(p.wd + (size_t)jj[u] * p.row_vecs + v);
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      if (u < cnt) {
#pragma unroll
        for (int b = 0; b < B; b++) DT::axpy(wv[u], s_z[b * p.chunk + jj[u] - j0], acc[b]);
      }
    }
  }

  CATS_STAMP(2);
  // ---- 3. fold the waves through LDS; slab partial -> scratch (y_out) or atomics (y32) ---------------------
  float* mypart = p.partial + ((size_t)slab * p.ngroup + group) * B * kSlabCols;
#pragma unroll
  for (int b = 0; b < B; b++) {
    if (b < p.nb) {  // uniform
#pragma unroll
      for (int e = 0; e < VEC; e++) s_red[wave * kSlabCols + e * kWave + lane] = acc[b][e];
      __syncthreads();
      for (int c = tid; c < kSlabCols; c += blockDim.x) {
        // c = e * 64 + l  ->  column (slab*64 + l) * VEC + e
        float s = 0.f;
        for (int w = 0; w < nwaves; w++) s += s_red[w * kSlabCols + c];
        if (p.y_out) {
          __hip_atomic_store(&mypart[b * kSlabCols + c], s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
          const int e = c >> 6, l = c & 63;
          const int col = (slab * kWave + l) * VEC + e;
          if (col < p.H && n > 0) unsafeAtomicAdd(&p.y32[(size_t)b * p.H + col], s);
        }
      }
      __syncthreads();
    }
  }

  if (p.count_out && blockIdx.x == 0) {  // not on the hot path: total popcount of the mask
    int k = 0;
    for (int byte = tid; byte * 8 < p.I; byte += blockDim.x) {
      uint32_t bits = p.mask[byte];
      const int rem = p.I - byte * 8;
      if (rem < 8) bits &= (1u << rem) - 1u;
      k += __popc(bits);
    }
    k = (int)wave_sum((float)k);  // far below 2^24: exact in fp32
    if (lane == 0) s_red[wave] = (float)k;
    __syncthreads();
    if (tid == 0) {
      float tot = 0.f;
      for (int w = 0; w < nwaves; w++) tot += s_red[w];
      *p.count_out = (int)tot;
    }
    __syncthreads();
  }
  CATS_STAMP(3);
  if (p.y_out == nullptr) return;

  // ---- 4. last workgroup of the slab adds the partials in group order and writes y ---------------------------
  // Ordering without a release / acquire fence pair (at agent scope those write back and invalidate the whole
  // L2 of the XCD, which costs far more than this kernel): partials are written and read with agent-scope
  // atomic stores / loads, which are coherent across the device by themselves.  Each wave waits until its own
  // stores have been acknowledged (s_waitcnt vmcnt(0)), the barrier joins the waves, and only then is the slab
  // counter bumped -- so when a workgroup reads "I am last" every partial of the slab is in place, and the loads
  // below, issued after that read, see them.
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), expcnt / lgkmcnt untouched
  __syncthreads();
  CATS_STAMP(4);
  if (tid == 0) {
    const uint32_t prev = __hip_atomic_fetch_add(&p.done[slab], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = prev == (uint32_t)p.ngroup - 1u;
  }
  __syncthreads();
  CATS_STAMP(5);
  if (!s_last) return;
  const float* slabpart = p.partial + (size_t)slab * p.ngroup * B * kSlabCols;
  for (int b = 0; b < p.nb; b++) {
    for (int c = tid; c < kSlabCols; c += blockDim.x) {
      const int e = c >> 6, l = c & 63;
      const int col = (slab * kWave + l) * VEC + e;
      float s = 0.f;
      for (int g0 = 0; g0 < p.ngroup; g0 += 8) {  // 8 independent loads in flight, added in group order
        float t[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
          const int gg = min(g0 + u, p.ngroup - 1);
          t[u] = __hip_atomic_load(&slabpart[((size_t)gg * B + b) * kSlabCols + c], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int u = 0; u < 8; u++)
          if (g0 + u < p.ngroup) s += t[u];
      }
      if (col < p.H) ((st*)p.y_out)[(size_t)b * p.H + col] = DT::fromf(s);
    }
  }
  if (tid == 0) __hip_atomic_store(&p.done[slab], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __builtin_amdgcn_s_waitcnt(0x0F70);
  CATS_STAMP(6);
}

}  // namespace cats
