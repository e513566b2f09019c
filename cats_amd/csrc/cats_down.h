// Sparse down projection over neuron-major weights: y[b,:] = sum over active j of z[b,j] * wdown_t[j,:].
//
// Work split.  Columns are cut into slabs of 64 lanes x 16 bytes (512 fp16 columns = 1 KiB of a row), the
// neurons into `ngroup` equal index ranges.  Workgroup (slab, group) streams the 1 KiB slab segment of every
// active row in its range: the waves deal the active rows round-robin and keep up to U loads in flight per
// lane.  Partial sums stay in registers (VEC per lane per batch row) and are folded across the waves of the
// workgroup through LDS.  Across workgroups there are two ways out:
//   * y_out (dtype output): every workgroup stores its partial sums to scratch, [group][b][H]; the reduction launch
//     that follows (reduce_partials_kernel) adds the ngroup partials in group order and writes the rounded result.
//     No atomics on data (32 workgroups adding into the same 16 cache lines serialise for microseconds), a fixed
//     summation order (bitwise reproducible output), nothing to zero between calls, no synchronisation between
//     workgroups other than the launch boundary.
//   * y32 (caller's fp32 accumulator, "atomic_gemv" semantics): one fp32 atomic per column per workgroup -- up to two
//     batch rows, where saving the second launch is worth it; from three rows on the partial sums go the first way and
//     the reduction launch adds their total into the accumulator.
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
  const uint8_t* mask;    // ceil(I/8) bytes, bit j = neuron j active for some batch row; or, with mask_bytes set, one
  int mask_bytes;         //   byte per neuron (readable up to the next multiple of eight), nonzero = active
  const uint8_t* flags;   // alternative to mask: (nb, I) flag bytes, OR-ed over the batch on the fly; NULL = use mask
  const int64_t* idx;     // alternative to both: an index list of M weight rows (any order, duplicates add up, entries outside
  int M;                  //   [0, I) contribute nothing); z is then (nb, M), aligned with the list, and the groups split the list
  float* y32;             // (nb, H) the caller's fp32 accumulator, added to with atomics when partial_out is not set
  void* y_out;            // (nb, H) dtype
  int partial_out;        // the folded sums go to `partial` and reduce_partials_kernel finishes (into y_out, or adds into y32)
  float* partial;         // [ngroup][nb][H] fp32 partial sums
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

// First phase of both down kernels.  Wave 0 turns the mask bytes (or flag bytes, or the given index list) of the range
// [j0, j1) into an ascending list of weight rows in s_list and leaves their number in *s_n; the other waves copy z of the
// range, rounded to the storage type, to s_z[b * chunk + (j - j0)] and zero rows nb .. zrows - 1.  The two loads are
// independent, so the phase costs one memory round trip.  The caller synchronises afterwards.
template <class DT, bool ZF32>
__device__ __forceinline__ void down_stage_list_and_z(const DownArgs& p, int j0, int j1, int zcols, bool by_list, int zrows, int* s_list,
                                                      typename DT::st* s_z, int* s_n) {
  typedef typename DT::st st;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  if (wave == 0 && by_list) {
    // the list is given: entry i of the range is weight row idx[j0 + i]
    for (int i = lane; i < j1 - j0; i += kWave) {
      const long long j = p.idx[j0 + i];
      s_list[i] = (j >= 0 && j < (long long)p.I) ? (int)j : 0;  // an entry outside the matrix reads row 0 against z = 0
    }
    if (lane == 0) *s_n = max(j1 - j0, 0);
  } else if (wave == 0) {
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
        } else if (p.mask_bytes) {  // uniform
          const uint2 m8 = *(const uint2*)(p.mask + (size_t)byte * 8);
#pragma unroll
          for (int e = 0; e < 4; e++) {
            bits |= ((m8.x >> (8 * e)) & 0xffu) ? 1u << e : 0u;
            bits |= ((m8.y >> (8 * e)) & 0xffu) ? 16u << e : 0u;
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
    if (lane == 0) *s_n = base;
  } else {
    // one flat loop over (b, q) so that the loads of all batch rows are in flight together
    const int span = j1 - j0;
    const int total = p.nb * span;
    for (int i = tid - kWave; i < total; i += blockDim.x - kWave) {
      const int b = i / span, q = i - b * span;
      const size_t o = (size_t)b * zcols + j0 + q;
      st zv = ZF32 ? DT::fromf(((const float*)p.z)[o]) : ((const st*)p.z)[o];
      if (by_list) {
        const long long j = p.idx[j0 + q];
        if (!(j >= 0 && j < (long long)p.I)) zv = DT::fromf(0.f);
      }
      s_z[b * p.chunk + q] = zv;
    }
    for (int i = p.nb * p.chunk + tid - kWave; i < zrows * p.chunk; i += blockDim.x - kWave) s_z[i] = DT::fromf(0.f);
  }
}

// Total popcount of the mask, by one workgroup (not on the hot path).  s_tmp: 16 floats of LDS nobody else is using.
__device__ __forceinline__ void down_count_mask(const DownArgs& p, float* s_tmp) {
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  int k = 0;
  if (p.mask_bytes) {
    for (int j = tid; j < p.I; j += blockDim.x) k += p.mask[j] != 0;
  } else {
    for (int byte = tid; byte * 8 < p.I; byte += blockDim.x) {
      uint32_t bits = p.mask[byte];
      const int rem = p.I - byte * 8;
      if (rem < 8) bits &= (1u << rem) - 1u;
      k += __popc(bits);
    }
  }
  k = (int)wave_sum((float)k);  // far below 2^24: exact in fp32
  if (lane == 0) s_tmp[wave] = (float)k;
  __syncthreads();
  if (tid == 0) {
    float tot = 0.f;
    for (int w = 0; w < (int)(blockDim.x >> 6); w++) tot += s_tmp[w];
    *p.count_out = (int)tot;
  }
}

template <class DT, int B, bool ZF32, int U>
__global__ __launch_bounds__(1024) void down_kernel(DownArgs p) {
  typedef typename DT::st st;
  constexpr int VEC = DT::VEC;
  constexpr int kSlabCols = kWave * VEC;
  constexpr int UP = U / 2;  // row pairs in flight per lane
  constexpr bool kPacked = sizeof(st) == 2;  // 16-bit types: z of a row pair travels as one packed dword
  extern __shared__ __attribute__((aligned(16))) float s_dyn[];  // 8- and 16-byte LDS accesses below: a 4-byte-aligned base makes every one of them a slow unaligned access
  // dynamic LDS, streaming phase: [chunk] int list | [B][chunk] z in storage type (indexed by j - j0)
  //                               | 16-bit types: [chunk / 2][B] packed z pairs in list order
  // afterwards reused for the fold: [nwaves][min(B, 4)][64][VEC] float
  int* s_list = (int*)s_dyn;
  st* s_z = (st*)(s_dyn + p.chunk);
  uint32_t* s_zp = (uint32_t*)(s_dyn + p.chunk) + (B * p.chunk * sizeof(st) + 3) / 4;
  float* s_red = s_dyn;
  __shared__ int s_n;

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform by construction; say so
  const int nwaves = blockDim.x >> 6;                         // a power of two
  const int slab = blockIdx.x % p.nslab;
  const int group = blockIdx.x / p.nslab;
  const bool by_list = p.idx != nullptr;          // uniform
  const int zcols = by_list ? p.M : p.I;          // row length of z
  const int j0 = group * p.chunk;                 // first neuron (or list position) of this group
  const int j1 = min(j0 + p.chunk, zcols);
  CATS_STAMP(0);

  // ---- 1. wave 0: mask bytes of the range -> ascending index list; the other waves: z of the range -> LDS ----
  down_stage_list_and_z<DT, ZF32>(p, j0, j1, zcols, by_list, B, s_list, s_z, &s_n);
  __syncthreads();
  const int n = s_n;
  const int nfull = n >> 1;  // whole pairs; pair k is list entries 2k and 2k + 1
  if (kPacked) {
    for (int i = tid; i < nfull * B; i += blockDim.x) {
      const int k = i / B, b = i - k * B;
      // z of a list entry sits at its neuron's offset in the range, or (index-list mode) at its position in the list
      const uint32_t za = s_z[b * p.chunk + (by_list ? 2 * k : s_list[2 * k] - j0)];
      const uint32_t zb = s_z[b * p.chunk + (by_list ? 2 * k + 1 : s_list[2 * k + 1] - j0)];
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
        else PairAxpy<DT, B>::run(wa[u], wb[u], s_z + (by_list ? 2 * kk[u] : ja[u] - j0), s_z + (by_list ? 2 * kk[u] + 1 : jb[u] - j0), p.chunk, acc);
      }
    }
  }
  if ((n & 1) && wave == nfull % nwaves) {  // odd list: the last row has no partner
    const int j = __builtin_amdgcn_readfirstlane(s_list[n - 1]);
    const u32x4 w = load_stream(p.wd + (size_t)j * p.row_vecs + v);
#pragma unroll
    for (int b = 0; b < B; b++) DT::axpy(w, DT::tof(s_z[b * p.chunk + (by_list ? n - 1 : j - j0)]), acc[b]);
  }

  CATS_STAMP(2);
  // ---- 3. fold the waves through LDS -----------------------------------------------------------------------
  // Up to four batch rows at a time (16 waves x 4 x 2 KiB = 128 KiB of LDS): every wave writes its sums, one barrier,
  // one thread per four columns adds the waves in wave order.  Eight batch rows take two such passes.  LDS layout of a
  // pass: the VEC sums of (wave w, row b, lane l) are the VEC / 4 float4 slots at ((w * FB + b) * 64 + l) * VEC / 4; for
  // 16-bit types (two slots per lane) the two halves swap places in lanes 8..15 of every 16, which makes both the
  // 16-byte writes (lane stride 32 bytes) and the reads (consecutive threads, consecutive slots) free of bank conflicts.
  // y_out mode: the folded sums go to the scratch partial [group][b][H]; the reduction launch that follows adds the
  // groups in order (a fixed summation order: bitwise reproducible output, nothing to zero between calls, no
  // cross-workgroup synchronisation inside this kernel).  y32 mode (the caller's fp32 accumulator, "atomic_gemv"
  // semantics): one fp32 atomic per column per workgroup.
  constexpr int FB = B < 4 ? B : 4;  // batch rows folded per pass
  constexpr int kSlots = VEC / 4;    // float4 slots per lane and batch row
  __syncthreads();  // the list and z are dead from here on; their LDS is reused
  CATS_STAMP(4);
  float4* s_red4 = (float4*)s_red;
#pragma unroll
  for (int b0 = 0; b0 < B; b0 += FB) {
    if (b0 > 0) __syncthreads();  // the previous pass has been read
    {
      const int swz = kSlots == 2 ? (lane >> 3) & 1 : 0;
#pragma unroll
      for (int b = 0; b < FB; b++)
#pragma unroll
        for (int h = 0; h < kSlots; h++) {
          float4 v4 = {acc[b0 + b][4 * h], acc[b0 + b][4 * h + 1], acc[b0 + b][4 * h + 2], acc[b0 + b][4 * h + 3]};
          s_red4[((size_t)(wave * FB + b) * kWave + lane) * kSlots + (h ^ swz)] = v4;
        }
    }
    __syncthreads();
    const int rows = min(FB, p.nb - b0);  // live batch rows of this pass (may be <= 0)
    // One item = one slot = four consecutive columns of one batch row: one float4 per wave from LDS, one 16-byte store.
    // Consecutive threads take consecutive slots, so whole 32-byte sectors are written by neighbouring lanes (a store
    // of part of a sector makes the memory side read the sector first).
    constexpr int kQuads = kSlabCols / 4;
    for (int it = tid; it < rows * kQuads; it += blockDim.x) {
      const int b = it / kQuads, r = it - b * kQuads;
      const int l = r / kSlots, ps = r - l * kSlots;                 // lane that owned the columns, physical slot
      const int h = kSlots == 2 ? ps ^ ((l >> 3) & 1) : ps;          // which quarter of its VEC the slot holds
      const float4* src = s_red4 + (size_t)b * kQuads + r;
      float4 s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
      for (int w = 0; w < nwaves; w++) {
        const float4 v4 = src[(size_t)w * FB * kQuads];
        s4.x += v4.x; s4.y += v4.y; s4.z += v4.z; s4.w += v4.w;
      }
      const int col = (slab * kWave + l) * VEC + 4 * h;
      if (col < p.H) {  // H is a multiple of VEC, so a quad is inside or outside as a whole
        if (p.partial_out) {
          *(float4*)&p.partial[((size_t)group * p.nb + b0 + b) * p.H + col] = s4;
        } else if (n > 0) {
          float* y = &p.y32[(size_t)(b0 + b) * p.H + col];
          unsafeAtomicAdd(y, s4.x); unsafeAtomicAdd(y + 1, s4.y); unsafeAtomicAdd(y + 2, s4.z); unsafeAtomicAdd(y + 3, s4.w);
        }
      }
    }
  }

  CATS_STAMP(5);
  if (p.count_out && blockIdx.x == 0) {  // not on the hot path: total popcount of the mask
    __syncthreads();  // s_red is reused below; the fold above may still be reading it
    down_count_mask(p, s_red);
  }
  CATS_STAMP(3);
}

}  // namespace cats
