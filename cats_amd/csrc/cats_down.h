// Sparse down projection over neuron-major weights: y[b,:] = sum over active j of z[b,j] * wdown_t[j,:].
//
// Work split.  Columns are cut into slabs of 64 lanes x 16 bytes (512 fp16 columns = 1 KiB of a row), the
// active neurons into `ngroup` equal runs of the ascending active list.  Workgroup (slab, group) streams
// the 1 KiB slab segment of every row in its run: each wave owns a subset of the run and keeps U loads in
// flight per lane.  Partial sums stay in registers (VEC per lane per batch row), are folded across the
// waves of the workgroup through LDS, and leave the workgroup as one fp32 atomic per column -- so the
// number of atomics is ngroup * H * B, independent of the number of waves.  blockIdx % nslab picks the
// slab, so with 8 slabs every XCD (workgroups are dealt round-robin over the 8 XCDs) streams one slab and
// all atomics on a given column come from one XCD.
//
// The active list is not read from memory: every workgroup rebuilds it from the mask words (popcount +
// block prefix sum), keeps the run it owns in LDS together with the matching z values, and goes on.
#pragma once
#include "cats_device.h"

namespace cats {

struct DownArgs {
  const u32x4* wd;        // (I, H) neuron-major
  const void* z;          // (nb, I) fp32 or dtype
  const uint64_t* mask;   // ceil(I/64) words, bit j = neuron j active for some batch row
  float* y32;             // (nb, H) fp32 accumulator: workspace (finalize) or the caller's buffer
  void* y_out;            // (nb, H) dtype; NULL => leave the sums in y32
  uint32_t* done;         // per-slab arrival counters (finalize only), zero between calls
  int32_t* count_out;     // optional: number of active neurons
  int H, I, nb;
  int row_vecs;           // H / VEC
  int nslab, ngroup, nwords;
  int ncap;               // LDS capacity (neurons) of one run
};

template <class DT, int B, bool ZF32, int U>
__global__ __launch_bounds__(1024) void down_kernel(DownArgs p) {
  typedef typename DT::st st;
  constexpr int VEC = DT::VEC;
  extern __shared__ float s_dyn[];
  // dynamic LDS: [ncap] int list | [B][ncap] float z | [nwaves][64*VEC] float partials
  int* s_list = (int*)s_dyn;
  float* s_z = s_dyn + p.ncap;
  float* s_red = s_z + (size_t)B * p.ncap;
  __shared__ int s_wsum[16];
  __shared__ int s_base;
  __shared__ int s_last;

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int nwaves = blockDim.x >> 6;
  const int slab = blockIdx.x % p.nslab;
  const int group = blockIdx.x / p.nslab;

  // ---- 1. popcount prefix over the mask words; expand this workgroup's run into LDS -------------
  // Two passes over the words: the first only counts (total k), the second places indices.
  int k = 0;
  for (int w0 = 0; w0 < p.nwords; w0 += blockDim.x) {
    const int w = w0 + tid;
    uint64_t word = 0;
    if (w < p.nwords) {
      word = p.mask[w];
      const int rem = p.I - w * 64;
      if (rem < 64) word &= (1ull << rem) - 1ull;
    }
    k += __popcll(word);
  }
  k = (int)wave_sum((float)k);  // counts are far below 2^24, exact in fp32
  if (lane == 0) s_wsum[wave] = k;
  __syncthreads();
  k = 0;
  for (int w = 0; w < nwaves; w++) k += s_wsum[w];
  const int lo = (int)(((long long)group * k) / p.ngroup);
  const int hi = (int)(((long long)(group + 1) * k) / p.ngroup);
  const int n = hi - lo;
  if (tid == 0) s_base = 0;
  __syncthreads();

  for (int w0 = 0; w0 < p.nwords; w0 += blockDim.x) {
    const int w = w0 + tid;
    uint64_t word = 0;
    if (w < p.nwords) {
      word = p.mask[w];
      const int rem = p.I - w * 64;
      if (rem < 64) word &= (1ull << rem) - 1ull;
    }
    const int pc = __popcll(word);
    const int incl = wave_scan_inclusive(pc, lane);
    if (lane == kWave - 1) s_wsum[wave] = incl;
    __syncthreads();
    int before = s_base;
    for (int ww = 0; ww < wave; ww++) before += s_wsum[ww];
    int rank = before + incl - pc;  // rank of this word's first set bit
    if (rank < hi && rank + pc > lo) {
      while (word) {
        const int bit = __builtin_ctzll(word);
        word &= word - 1;
        if (rank >= lo && rank < hi) s_list[rank - lo] = w * 64 + bit;
        rank++;
      }
    }
    __syncthreads();
    if (tid == 0) {
      int tot = s_base;
      for (int ww = 0; ww < nwaves; ww++) tot += s_wsum[ww];
      s_base = tot;
    }
    __syncthreads();
  }
  // stage z for the run
  for (int i = tid; i < n * B; i += blockDim.x) {
    const int b = i / n, q = i - b * n;
    float zv = 0.f;
    if (b < p.nb) {
      const size_t o = (size_t)b * p.I + s_list[q];
      zv = ZF32 ? ((const float*)p.z)[o] : DT::tof(((const st*)p.z)[o]);
    }
    s_z[b * p.ncap + q] = zv;
  }
  __syncthreads();

  // ---- 2. stream the slab segments of the run -----------------------------------------------------
  float acc[B][VEC];
#pragma unroll
  for (int b = 0; b < B; b++)
#pragma unroll
    for (int e = 0; e < VEC; e++) acc[b][e] = 0.f;

  // Lanes past the end of a row (H not a multiple of 64 * VEC) re-read the row's last vector; their sums
  // are dropped at the column check below, so no load is predicated and U of them stay in flight.
  const int v = min(slab * kWave + lane, p.row_vecs - 1);
  for (int i0 = wave * U; i0 < n; i0 += nwaves * U) {
    u32x4 wv[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int j = s_list[min(i0 + u, n - 1)];
      wv[u] = load_stream(p.wd + (size_t)j * p.row_vecs + v);
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      const bool live = i0 + u < n;  // wave-uniform
      const int q = live ? i0 + u : 0;
#pragma unroll
      for (int b = 0; b < B; b++) {
        const float zq = live ? s_z[b * p.ncap + q] : 0.f;
        DT::axpy(wv[u], zq, acc[b]);
      }
    }
  }

  // ---- 3. fold the waves through LDS, one atomic per column ----------------------------------------
  constexpr int kSlabCols = kWave * VEC;
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
        const int e = c >> 6, l = c & 63;
        const int col = (slab * kWave + l) * VEC + e;
        if (col < p.H && n > 0) unsafeAtomicAdd(&p.y32[(size_t)b * p.H + col], s);
      }
      __syncthreads();
    }
  }

  if (blockIdx.x == 0 && tid == 0 && p.count_out) *p.count_out = k;
  if (p.y_out == nullptr) return;

  // ---- 4. last workgroup of the slab rounds the sums into y and clears the accumulator ---------------
  __threadfence();
  __syncthreads();
  if (tid == 0) {
    const uint32_t prev = __hip_atomic_fetch_add(&p.done[slab], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    s_last = prev == (uint32_t)p.ngroup - 1u;
  }
  __syncthreads();
  if (!s_last) return;
  __threadfence();
  for (int i = tid; i < p.nb * kSlabCols; i += blockDim.x) {
    const int b = i / kSlabCols, c = i - b * kSlabCols;
    const int col = slab * kSlabCols + c;
    if (col < p.H) {
      const size_t o = (size_t)b * p.H + col;
      const float s = __hip_atomic_exchange(&p.y32[o], 0.f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      ((st*)p.y_out)[o] = DT::fromf(s);
    }
  }
  if (tid == 0) __hip_atomic_store(&p.done[slab], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace cats
