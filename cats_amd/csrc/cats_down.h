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
  const uint8_t* flags;   // alternative to mask: (nb, I) flag bytes, OR-ed over the batch on the fly; NULL = use mask
  float* y32;             // (nb, H) the caller's fp32 accumulator (atomics), used when y_out == NULL
  void* y_out;            // (nb, H) dtype
  const void* residual;   // optional (nb, H) dtype, y_out mode: y = residual + round(sum); may alias y_out
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

// Adds z-weighted weight vectors of two active rows into acc[b][0..VEC).  16-bit types interleave the two rows
// element-wise (one v_perm per dword) so that one v_dot2 per column does both rows; fp32 is two plain axpy.
template <class DT, int B>
struct PairAxpy {
  typedef typename DT::st st;
  static __device__ __forceinline__ void run(u32x4 wa, u32x4 wb, const st* za, const st* zb, int zstride, float (*acc)[DT::VEC]) {
#pragma unroll
    for (int b = 0; b < B; b++) {
      DT::axpy(wa, DT::tof(za[b * zstride]), acc[b]);
      DT::axpy(wb, DT::tof(zb[b * zstride]), acc[b]);
    }
  }
};

template <class DT, int B>
struct PairAxpy16 {
  // zp[b] = (z[b, row a], z[b, row b]) packed in storage type; a missing second row has weight and z zero
  static __device__ __forceinline__ void run(u32x4 wa, u32x4 wb, const uint32_t* zp, float (*acc)[8]) {
    uint32_t lo[4], hi[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      lo[i] = __builtin_amdgcn_perm(wb[i], wa[i], 0x05040100u);  // (wa[i].lo16, wb[i].lo16): column 2i of both rows
      hi[i] = __builtin_amdgcn_perm(wb[i], wa[i], 0x07060302u);  // (wa[i].hi16, wb[i].hi16): column 2i + 1
    }
#pragma unroll
    for (int b = 0; b < B; b++) {
      const uint32_t z2 = zp[b];
#pragma unroll
      for (int i = 0; i < 4; i++) {
        acc[b][2 * i] = DT::dot2(lo[i], z2, acc[b][2 * i]);
        acc[b][2 * i + 1] = DT::dot2(hi[i], z2, acc[b][2 * i + 1]);
      }
    }
  }
};

template <class DT, int B, bool ZF32, int U>
__global__ __launch_bounds__(1024) void down_kernel(DownArgs p) {
  typedef typename DT::st st;
  constexpr int VEC = DT::VEC;
  constexpr int kSlabCols = kWave * VEC;
  constexpr int UP = U / 2;  // row pairs in flight per lane
  constexpr bool kPacked = sizeof(st) == 2;  // 16-bit types: z of a row pair travels as one packed dword
  extern __shared__ float s_dyn[];
  // dynamic LDS, streaming phase: [chunk] int list | [B][chunk] z in storage type (indexed by j - j0)
  //                               | 16-bit types: [chunk / 2][B] packed z pairs in list order
  // afterwards reused for the fold: [nwaves / 2][B][VEC][64] float
  int* s_list = (int*)s_dyn;
  st* s_z = (st*)(s_dyn + p.chunk);
  uint32_t* s_zp = (uint32_t*)(s_dyn + p.chunk) + (B * p.chunk * sizeof(st) + 3) / 4;
  float* s_red = s_dyn;
  __shared__ int s_n;
  __shared__ int s_last;

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform by construction; say so
  const int nwaves = blockDim.x >> 6;                         // a power of two
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
        if (p.flags) {  // uniform: per-row flag bytes instead of packed bits
          for (int e = 0; e < 8; e++) {
            const int j = byte * 8 + e;
            uint32_t on = 0;
            if (j < p.I)
              for (int b = 0; b < p.nb; b++) on |= p.flags[(size_t)b * p.I + j] != 0 ? 1u : 0u;
            bits |= on << e;
          }
        } else {
          bits = p.mask[byte];
        }
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
    // one flat loop over (b, q) so that the loads of all batch rows are in flight together
    const int span = j1 - j0;
    const int total = p.nb * span;
    for (int i = tid - kWave; i < total; i += blockDim.x - kWave) {
      const int b = i / span, q = i - b * span;
      const size_t o = (size_t)b * p.I + j0 + q;
      s_z[b * p.chunk + q] = ZF32 ? DT::fromf(((const float*)p.z)[o]) : ((const st*)p.z)[o];
    }
    for (int i = p.nb * p.chunk + tid - kWave; i < B * p.chunk; i += blockDim.x - kWave) s_z[i] = DT::fromf(0.f);
  }
  __syncthreads();
  const int n = s_n;
  const int nfull = n >> 1;  // whole pairs; pair k is list entries 2k and 2k + 1
  if (kPacked) {
    for (int i = tid; i < nfull * B; i += blockDim.x) {
      const int k = i / B, b = i - k * B;
      const uint32_t za = s_z[b * p.chunk + s_list[2 * k] - j0], zb = s_z[b * p.chunk + s_list[2 * k + 1] - j0];
      s_zp[i] = za | (zb << 16);
    }
    __syncthreads();
  }
  CATS_STAMP(1);

  // ---- 2. stream the slab segments of the active rows, two rows at a time --------------------------------
  float acc[B][VEC];
#pragma unroll
  for (int b = 0; b < B; b++)
#pragma unroll
    for (int e = 0; e < VEC; e++) acc[b][e] = 0.f;

  // Lanes past the end of a row (H not a multiple of 64 * VEC) re-read the row's last vector; their sums
  // are dropped at the column check below, so no load is predicated per lane.
  const int v = min(slab * kWave + lane, p.row_vecs - 1);
  // This wave owns pairs wave, wave + nwaves, ...; split them into passes of at most UP, evenly.
  const int mine = nfull > wave ? (nfull - wave + nwaves - 1) / nwaves : 0;
  const int passes = (mine + UP - 1) / UP;
  const int per = passes ? (mine + passes - 1) / passes : 0;
  for (int t0 = 0; t0 < mine; t0 += per) {
    const int cnt = min(per, mine - t0);  // wave-uniform
    u32x4 wa[UP], wb[UP];
    int kk[UP], ja[UP], jb[UP];
#pragma unroll
    for (int u = 0; u < UP; u++) {
      if (u < cnt) {
        kk[u] = wave + (t0 + u) * nwaves;
        ja[u] = __builtin_amdgcn_readfirstlane(s_list[2 * kk[u]]);
        jb[u] = __builtin_amdgcn_readfirstlane(s_list[2 * kk[u] + 1]);
        wa[u] = load_stream(p.wd + (size_t)ja[u] * p.row_vecs + v);
        wb[u] = load_stream(p.wd + (size_t)jb[u] * p.row_vecs + v);
      }
    }
#pragma unroll
    for (int u = 0; u < UP; u++) {
      if (u < cnt) {
        if constexpr (kPacked) PairAxpy16<DT, B>::run(wa[u], wb[u], s_zp + kk[u] * B, acc);
        else PairAxpy<DT, B>::run(wa[u], wb[u], s_z + (ja[u] - j0), s_z + (jb[u] - j0), p.chunk, acc);
      }
    }
  }
  if ((n & 1) && wave == nfull % nwaves) {  // odd list: the last row has no partner
    const int j = __builtin_amdgcn_readfirstlane(s_list[n - 1]);
    const u32x4 w = load_stream(p.wd + (size_t)j * p.row_vecs + v);
#pragma unroll
    for (int b = 0; b < B; b++) DT::axpy(w, DT::tof(s_z[b * p.chunk + j - j0]), acc[b]);
  }

  CATS_STAMP(2);
  // ---- 3. fold the waves through LDS -----------------------------------------------------------------------
  // Up to four batch rows (16 waves x 4 x 2 KiB = 128 KiB of LDS): every wave writes its sums, one barrier, one thread per column adds the waves in wave
  // order and stores the slab partial.  More batch rows would not fit in LDS that way: pairwise rounds instead
  // (upper half writes, lower half adds), after which wave 0 holds the partial.
  // Partial layout (both ways): float (b, pair p, lane l, k) at b*kSlabCols + p*128 + l*2 + k  is column
  // (slab*64 + l) * VEC + 2p + k.
  float* mypart = p.partial + ((size_t)slab * p.ngroup + group) * B * kSlabCols;
  __syncthreads();  // the list and z are dead from here on; their LDS is reused
  if constexpr (B <= 4) {
    {
      float* dst = s_red + (size_t)wave * B * kSlabCols + lane * 2;
#pragma unroll
      for (int b = 0; b < B; b++)
#pragma unroll
        for (int e = 0; e < VEC; e += 2) {
          float2 v2 = {acc[b][e], acc[b][e + 1]};
          *(float2*)(dst + b * kSlabCols + (e >> 1) * (2 * kWave)) = v2;
        }
    }
    __syncthreads();
    for (int f = tid; f < p.nb * kSlabCols; f += blockDim.x) {
      float s = 0.f;
      for (int w = 0; w < nwaves; w++) s += s_red[(size_t)w * B * kSlabCols + f];
      if (p.y_out) {
        __hip_atomic_store(&mypart[f], s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      } else {
        const int b = f / kSlabCols, c = f - b * kSlabCols;
        const int col = (slab * kWave + ((c & (2 * kWave - 1)) >> 1)) * VEC + (c / (2 * kWave)) * 2 + (c & 1);
        if (col < p.H && n > 0) unsafeAtomicAdd(&p.y32[(size_t)b * p.H + col], s);
      }
    }
  } else {
    for (int half = nwaves >> 1; half >= 1; half >>= 1) {
      if (wave >= half && wave < 2 * half) {
        float* dst = s_red + (size_t)(wave - half) * B * kSlabCols;
#pragma unroll
        for (int b = 0; b < B; b++)
#pragma unroll
          for (int e = 0; e < VEC; e++) dst[(b * VEC + e) * kWave + lane] = acc[b][e];
      }
      __syncthreads();
      if (wave < half) {
        const float* src = s_red + (size_t)wave * B * kSlabCols;
#pragma unroll
        for (int b = 0; b < B; b++)
#pragma unroll
          for (int e = 0; e < VEC; e++) acc[b][e] += src[(b * VEC + e) * kWave + lane];
      }
      __syncthreads();
    }
    if (wave == 0) {
#pragma unroll
      for (int b = 0; b < B; b++) {
        if (b < p.nb) {  // uniform
          if (p.y_out) {
#pragma unroll
            for (int e = 0; e < VEC; e += 2) {
              const uint64_t two = (uint64_t)__float_as_uint(acc[b][e]) | ((uint64_t)__float_as_uint(acc[b][e + 1]) << 32);
              __hip_atomic_store((uint64_t*)&mypart[b * kSlabCols + (e >> 1) * (2 * kWave) + 2 * lane], two, __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
            }
          } else {
#pragma unroll
            for (int e = 0; e < VEC; e++) {
              const int col = (slab * kWave + lane) * VEC + e;
              if (col < p.H && n > 0) unsafeAtomicAdd(&p.y32[(size_t)b * p.H + col], acc[b][e]);
            }
          }
        }
      }
    }
  }

  if (p.count_out && blockIdx.x == 0) {  // not on the hot path: total popcount of the mask
    __syncthreads();  // s_red is reused below; the fold above may still be reading it
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
  // atomic stores / loads, which are coherent across the device by themselves.  Every wave waits until its own
  // stores have been acknowledged (s_waitcnt vmcnt(0)), the barrier joins them, and only then is the slab counter bumped -- so when a
  // workgroup reads "I am last" every partial of the slab is in place, and the loads below, issued after
  // that read, see them.
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), expcnt / lgkmcnt untouched: this wave's partial stores are acknowledged
  __syncthreads();                     // ... and so are everybody else's
  CATS_STAMP(4);
  if (tid == 0) {
    const uint32_t prev = __hip_atomic_fetch_add(&p.done[slab], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = prev == (uint32_t)p.ngroup - 1u;
  }
  __syncthreads();
  CATS_STAMP(5);
  if (!s_last) return;
  const uint64_t* slabpart = (const uint64_t*)(p.partial + (size_t)slab * p.ngroup * B * kSlabCols);
  constexpr int kPairs = VEC / 2 * kWave;  // 64-bit items per batch row and group
  constexpr int kInFlight = 32;  // with the default 32 groups every partial of an item is requested in one go
  for (int item = tid; item < p.nb * kPairs; item += blockDim.x) {
    const int b = item / kPairs, r = item - b * kPairs;
    const int e = (r >> 6) * 2, l = r & 63;
    const int col = (slab * kWave + l) * VEC + e;
    float s0 = 0.f, s1 = 0.f;
    for (int g0 = 0; g0 < p.ngroup; g0 += kInFlight) {  // independent loads in flight, added in group order
      uint64_t t[kInFlight];
#pragma unroll
      for (int u = 0; u < kInFlight; u++) {
        const int gg = min(g0 + u, p.ngroup - 1);
        t[u] = __hip_atomic_load(&slabpart[((size_t)gg * B + b) * kPairs + r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
#pragma unroll
      for (int u = 0; u < kInFlight; u++) {
        if (g0 + u < p.ngroup) {
          s0 += __uint_as_float((uint32_t)t[u]);
          s1 += __uint_as_float((uint32_t)(t[u] >> 32));
        }
      }
    }
    if (col < p.H) {
      st* y = (st*)p.y_out + (size_t)b * p.H + col;
      if (p.residual) {  // the MLP output is rounded to the storage type first, as a module returning a tensor would
        const st* res = (const st*)p.residual + (size_t)b * p.H + col;
        s0 = DT::rnd(s0) + DT::tof(res[0]);
        s1 = DT::rnd(s1) + DT::tof(res[1]);
      }
      y[0] = DT::fromf(s0);
      y[1] = DT::fromf(s1);
    }
  }
  if (tid == 0) __hip_atomic_store(&p.done[slab], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __builtin_amdgcn_s_waitcnt(0x0F70);
  CATS_STAMP(6);
}

}  // namespace cats
