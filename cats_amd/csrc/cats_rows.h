// Row-streaming kernel: one wavefront owns R consecutive weight rows at a time, every lane issues
// 128-bit streaming loads over the row, the dot products are accumulated in fp32 and folded across the
// wave with DPP.  One template covers the four row-major passes of the CATS MLP:
//
//   kGate    a = SiLU(x . wgate[j]) ; flag = |a| > t ; optional mask words ; optional compact list
//   kGateUp  the gate pass, then for rows that came out active the matching wup row:  z = a * (x . wup[j])
//   kUp      flags and a are given; fetch wup rows with any flag set:                  out = a * (x . wup[j])
//   kGemv    plain y = W x (the dense (H,I) down projection over the zero-filled intermediate)
//
// x is staged once per workgroup in LDS, zero-padded to a whole number of 64-lane vectors, and read back
// as one ds_read_b128 per lane per chunk (conflict-free: consecutive lanes, consecutive 16 bytes).
#pragma once
#include "cats_device.h"

namespace cats {

enum RowsMode { kGate = 0, kGateUp = 1, kUp = 2, kGemv = 3 };

struct RowsArgs {
  const u32x4* x;        // (B, K) activations (K = row length of w)
  const u32x4* w;        // (N, K) first weight: wgate (kGate, kGateUp), wup (kUp), W (kGemv)
  const u32x4* w2;       // (N, K) wup for kGateUp
  const void* a_in;      // kUp: (nb, N) gate activations in dtype
  const uint8_t* flag_in;  // kUp: (nb, N); NULL = derive the flags from a_in:  |a| > t
  void* a_out;           // kGate: (nb, N) dtype, optional
  uint8_t* flag_out;     // kGate, kGateUp: (nb, N), optional
  uint8_t* mask_out;     // kGate, kGateUp: ceil(N/8) bytes, bit j = OR over the batch of flag[b, j]; optional
  float* z32_out;        // kGateUp: (nb, N) fp32, written for rows fetched from wup only; kUp: fp32 out, all rows
  void* zt_out;          // kGateUp, kUp, kGemv: (nb, N) dtype, every row written (0 where inactive)
  // compact list, kGate with nb == 1 only
  uint32_t* arrive;      // zeroed counter; the last workgroup to finish builds the list and resets it
  uint32_t* arrive_sub;  // 64 zeroed counters, 128 bytes apart: first level of the arrival count
  int64_t* idx_out;
  void* vals_out;
  int32_t* count_out;
  int K;                 // row length in elements
  int N;                 // number of rows
  int nb;                // live batch rows (<= template B)
  int nch;               // 64-lane vector chunks per row: ceil(K / (64 * VEC))
  int row_vecs;          // K / VEC
  float t;               // threshold, already rounded through dtype
  int lds_floor;         // host side only: request at least this much dynamic LDS (caps workgroups per CU); 0 = none
  const u32x4* norm_w;   // optional (K,) RMS-norm weight: x is replaced by norm_w * round(x * rsqrt(mean(x^2) + norm_eps)) while
  float norm_eps;        //   it is staged (needs x in LDS); NULL = x is used as given
  int mma;               // host side only: kGateUp with 2..8 batch rows may take the matrix-core kernel
#ifdef CATS_TIMING
  long long* tbuf;       // [gridDim][8] wall-clock stamps (100 MHz) at phase boundaries, development builds only
#endif
};

#ifdef CATS_TIMING
#define CATS_RSTAMP(slot) do { if (p.tbuf && threadIdx.x == 0) p.tbuf[(size_t)blockIdx.x * 8 + (slot)] = wall_clock64(); } while (0)
#else
#define CATS_RSTAMP(slot) do { } while (0)
#endif

// One block of weight loads: CB chunks of 64 lanes x 16 bytes for each of the R rows, issued back to back so
// they are all in flight together.  Loads are never predicated per lane: lanes past the end of a row re-read
// its last vector and later meet a zero in x (the LDS copy of x is zero-padded to whole blocks of CB chunks).
template <int R, int CB, bool FULL>
__device__ __forceinline__ void rows_issue(const u32x4* __restrict__ w, const int (&row)[R], const bool (&on)[R], int c0,
                                           const RowsArgs& p, int lane, u32x4 (&wv)[R][CB]) {
  const int vlast = p.row_vecs - 1;
#pragma unroll
  for (int r = 0; r < R; r++) {
    if (on[r]) {  // wave-uniform
      const u32x4* wr = w + (size_t)row[r] * p.row_vecs;
#pragma unroll
      for (int cc = 0; cc < CB; cc++) {
        const int v = (c0 + cc) * kWave + lane;
        wv[r][cc] = load_stream(wr + (FULL ? v : min(v, vlast)));
      }
    } else {
      // defined on every path: inside a persistent loop an undefined value would stay live across iterations
#pragma unroll
      for (int cc = 0; cc < CB; cc++) wv[r][cc] = zero4();
    }
  }
}

// Dot products of R weight rows against the nb staged x rows.  acc[r][b] ends up wave-uniform.  `wv` holds the
// loads of the first block if `preissued` (the caller started them before x was staged), else it is scratch.
template <class DT, int B, int R, int CB, bool FULL, bool XLDS>
__device__ __forceinline__ void rows_dot(const u32x4* __restrict__ w, const int (&row)[R], const bool (&on)[R],
                                         const u32x4* xs, const u32x4* __restrict__ xg, const RowsArgs& p, int lane,
                                         u32x4 (&wv)[R][CB], bool preissued, float (&acc)[R][B]) {
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int b = 0; b < B; b++) acc[r][b] = 0.f;

  const int vlast = p.row_vecs - 1;
  const int nchp = (p.nch + CB - 1) / CB * CB;
  for (int c0 = 0; c0 < p.nch; c0 += CB) {
    if (!(preissued && c0 == 0)) rows_issue<R, CB, FULL>(w, row, on, c0, p, lane, wv);
#pragma unroll
    for (int cc = 0; cc < CB; cc++) {
      const int v = (c0 + cc) * kWave + lane;
#pragma unroll
      for (int b = 0; b < B; b++) {
        u32x4 xv;
        if (XLDS) {
          xv = xs[b * nchp * kWave + v];
        } else {
          xv = xg[(size_t)min(b, p.nb - 1) * p.row_vecs + min(v, vlast)];
          if (!(b < p.nb && v < p.row_vecs)) xv = zero4();
        }
#pragma unroll
        for (int r = 0; r < R; r++)
          if (on[r]) acc[r][b] = DT::dot(wv[r][cc], xv, acc[r][b]);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; r++)
    if (on[r]) {
#pragma unroll
      for (int b = 0; b < B; b++) acc[r][b] = wave_sum(acc[r][b]);
    }
}

// B == 1 asks for 6 waves per SIMD (80 VGPRs): 6 workgroups of 4 waves per CU hold all 1376 workgroups of an
// 11008-row matrix at once, so no workgroup starts late and runs its two dependent passes on a draining machine.
template <class DT, int B, int R, int CB, bool FULL, int MODE, bool XLDS, int WAVES>
__global__ __launch_bounds__(WAVES* kWave) __attribute__((amdgpu_waves_per_eu(B == 1 && WAVES == 4 && FULL ? 6 : 1, 8)))
void rows_kernel(RowsArgs p) {
  typedef typename DT::st st;
  extern __shared__ u32x4 xs[];  // [B][round_up(nch, CB) * 64] vectors (XLDS only)
  __shared__ uint32_t s_maskbits;
  __shared__ int s_last;
  __shared__ int s_wtot[WAVES];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform by construction; say so
  constexpr int kThreads = WAVES * kWave;
  constexpr int kRowsPerBlock = WAVES * R;
  static_assert(kRowsPerBlock % 8 == 0 && kRowsPerBlock <= 32, "mask bytes are assembled in one 32-bit LDS word");

  CATS_RSTAMP(0);
  const int row0 = (blockIdx.x * WAVES + wave) * R;
  int row[R];
  bool on[R];
#pragma unroll
  for (int r = 0; r < R; r++) {
    row[r] = row0 + r < p.N ? row0 + r : p.N - 1;
    on[r] = row0 + r < p.N;
  }

  // Staging order matters: memory returns are counted in issue order, so the x loads go out first, then the
  // first block of weight loads, and only the x values are waited for before the LDS writes and the barrier --
  // the weight loads stay in flight across both.
  u32x4 wv[R][CB];
  // x vectors per thread fetched ahead of the weights: all of x for H = 4096 in 16-bit types (B * 512 vectors)
  constexpr int kXPreAll = (B * 512 + kThreads - 1) / kThreads;
  constexpr int kXPre = kXPreAll < 4 ? kXPreAll : 4;  // more would spill at B = 8
  const int nchv = (p.nch + CB - 1) / CB * CB * kWave;  // padded vectors per x row
  u32x4 xpre[kXPre];
  if (XLDS) {
#pragma unroll
    for (int k = 0; k < kXPre; k++) {
      const int i = threadIdx.x + k * kThreads;
      const int b = B == 1 ? 0 : i / nchv, v = i - b * nchv;
      xpre[k] = zero4();
      if (i < B * nchv && b < p.nb && v < p.row_vecs) xpre[k] = p.x[(size_t)b * p.row_vecs + v];
    }
  }
  if (MODE != kUp) rows_issue<R, CB, FULL>(p.w, row, on, 0, p, lane, wv);
  if (XLDS) {
#pragma unroll
    for (int k = 0; k < kXPre; k++) {
      const int i = threadIdx.x + k * kThreads;
      if (i < B * nchv) xs[i] = xpre[k];
    }
    for (int i = threadIdx.x + kXPre * kThreads; i < B * nchv; i += kThreads) {
      const int b = i / nchv, v = i - b * nchv;
      u32x4 val = zero4();
      if (b < p.nb && v < p.row_vecs) val = p.x[(size_t)b * p.row_vecs + v];
      xs[i] = val;
    }
  }
  if (threadIdx.x == 0) s_maskbits = 0u;
  __syncthreads();
  if (XLDS && p.norm_w) {
    // RMS norm of each batch row, in place in LDS: one wave adds a row's squares (fixed order), everyone rescales.
    __shared__ float s_scale[B];
    for (int b = wave; b < B; b += WAVES) {
      float ss = 0.f;
      for (int v = lane; v < p.row_vecs; v += kWave) ss = vec_sumsq<DT>(xs[b * nchv + v], ss);
      ss = wave_sum(ss);
      if (lane == 0) s_scale[b] = rsqrtf(ss / (float)p.K + p.norm_eps);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < B * nchv; i += kThreads) {
      const int b = B == 1 ? 0 : i / nchv, v = i - b * nchv;
      if (b < p.nb && v < p.row_vecs) xs[i] = vec_norm_apply<DT>(xs[i], s_scale[b], p.norm_w[v]);
    }
    __syncthreads();
  }
  CATS_RSTAMP(1);

  float a[R][B];       // gate activation, rounded through dtype
  bool act[R][B];      // per batch row flag
  bool any[R];         // union over the batch

  if (MODE == kUp) {
    const st* ain = (const st*)p.a_in;
#pragma unroll
    for (int r = 0; r < R; r++) {
      any[r] = false;
#pragma unroll
      for (int b = 0; b < B; b++) {
        const bool live = on[r] && b < p.nb;
        const float av = live ? DT::tof(ain[(size_t)b * p.N + row[r]]) : 0.f;
        act[r][b] = live && (p.flag_in ? p.flag_in[(size_t)b * p.N + row[r]] != 0 : fabsf(av) > p.t);
        a[r][b] = act[r][b] ? av : 0.f;
        any[r] = any[r] || act[r][b];
      }
      // flags are per-lane loads of the same address; make the branch below provably wave-uniform
      any[r] = __builtin_amdgcn_readfirstlane((int)any[r]) != 0;
    }
    if (p.mask_out && lane == 0) {
      uint32_t bits = 0u;
#pragma unroll
      for (int r = 0; r < R; r++) bits |= (any[r] ? 1u : 0u) << (wave * R + r);
      if (bits) atomicOr(&s_maskbits, bits);
    }
  } else {
    float g[R][B];
    rows_dot<DT, B, R, CB, FULL, XLDS>(p.w, row, on, xs, p.x, p, lane, wv, true, g);
    if (MODE == kGemv) {
      if (lane == 0) {
        st* out = (st*)p.zt_out;
#pragma unroll
        for (int r = 0; r < R; r++)
          if (on[r]) {
#pragma unroll
            for (int b = 0; b < B; b++)
              if (b < p.nb) out[(size_t)b * p.N + row[r]] = DT::fromf(g[r][b]);
          }
      }
      return;
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
      any[r] = false;
#pragma unroll
      for (int b = 0; b < B; b++) {
        const float gr = DT::rnd(g[r][b]);
        a[r][b] = DT::rnd(gr / (1.f + expf(-gr)));
        act[r][b] = on[r] && b < p.nb && fabsf(a[r][b]) > p.t;
        any[r] = any[r] || act[r][b];
      }
    }
    if (lane == 0) {
#pragma unroll
      for (int r = 0; r < R; r++)
        if (on[r]) {
#pragma unroll
          for (int b = 0; b < B; b++)
            if (b < p.nb) {
              if (MODE == kGate && p.a_out) {
                st* dst = (st*)p.a_out + (size_t)b * p.N + row[r];
                // read back by another workgroup (the one that builds the list): device-coherent store
                if (p.idx_out) __hip_atomic_store(dst, DT::fromf(a[r][b]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                else *dst = DT::fromf(a[r][b]);
              }
              if (p.flag_out) p.flag_out[(size_t)b * p.N + row[r]] = act[r][b] ? 1 : 0;
            }
        }
      if (p.mask_out) {
        uint32_t bits = 0u;
#pragma unroll
        for (int r = 0; r < R; r++) bits |= (any[r] ? 1u : 0u) << (wave * R + r);
        if (bits) atomicOr(&s_maskbits, bits);
      }
    }
  }

  CATS_RSTAMP(2);
  if (MODE == kGateUp || MODE == kUp) {
    float u[R][B];
    rows_dot<DT, B, R, CB, FULL, XLDS>(MODE == kGateUp ? p.w2 : p.w, row, any, xs, p.x, p, lane, wv, false, u);
    if (lane == 0) {
#pragma unroll
      for (int r = 0; r < R; r++)
        if (on[r]) {
#pragma unroll
          for (int b = 0; b < B; b++)
            if (b < p.nb) {
              const float z = act[r][b] ? DT::rnd(a[r][b] * DT::rnd(u[r][b])) : 0.f;
              const size_t o = (size_t)b * p.N + row[r];
              if (p.z32_out && (MODE == kUp || any[r])) p.z32_out[o] = z;
              if (p.zt_out) ((st*)p.zt_out)[o] = DT::fromf(z);
            }
        }
    }
  }

  CATS_RSTAMP(3);
  if (MODE == kGate || MODE == kGateUp || MODE == kUp) {
    if (p.mask_out) {
      __syncthreads();
      const int nbytes = (p.N + 7) >> 3;
      if (threadIdx.x < kRowsPerBlock / 8) {
        const int byte = blockIdx.x * (kRowsPerBlock / 8) + threadIdx.x;
        if (byte < nbytes) {
          const uint8_t m8 = (uint8_t)(s_maskbits >> (8 * threadIdx.x));
          if (MODE == kGate && p.idx_out) __hip_atomic_store(&p.mask_out[byte], m8, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          else p.mask_out[byte] = m8;
        }
      }
    }
  }

  if (MODE == kGate) {
    if (p.idx_out == nullptr) return;
    // Last workgroup to arrive turns the mask bytes into an ascending index list: one byte (8 neurons) per thread
    // and pass, popcount + wave prefix sum + LDS prefix over the waves for the rank, bit expansion for the entries.
    // No release / acquire fences (at agent scope they write back and invalidate the whole L2): the activations and
    // mask bytes were stored device-coherently above, each wave waits for its own stores to be acknowledged, the
    // barrier joins the waves, then the arrival counter is bumped; the last workgroup reads with coherent loads.
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();
    if (threadIdx.x == 0) {
      // Two levels: atomics on one address are served one after the other (about 12 ns each), which for a thousand
      // workgroups would cost more than the gate pass.  Workgroups count into 64 counters on separate lines; the
      // last one of each counts into the top one.
      constexpr uint32_t kSub = 64;
      const uint32_t sub = blockIdx.x % kSub;
      const uint32_t members = (gridDim.x - sub + kSub - 1) / kSub;
      uint32_t* sc = p.arrive_sub + sub * 32;
      bool last = false;
      if (__hip_atomic_fetch_add(sc, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == members - 1u) {
        __hip_atomic_store(sc, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const uint32_t used = gridDim.x < kSub ? gridDim.x : kSub;
        last = __hip_atomic_fetch_add(p.arrive, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == used - 1u;
      }
      s_last = last;
    }
    __syncthreads();
    if (!s_last) return;
    const st* aall = (const st*)p.a_out;
    const int nbytes = (p.N + 7) >> 3;
    int base = 0;
    for (int b0 = 0; b0 < nbytes; b0 += kThreads) {
      const int byte = b0 + threadIdx.x;
      uint32_t bits = 0;
      if (byte < nbytes) bits = __hip_atomic_load(&p.mask_out[byte], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const int pc = __popc(bits);
      const int incl = wave_scan_inclusive(pc, lane);
      if (lane == kWave - 1) s_wtot[wave] = incl;
      __syncthreads();
      int before = 0, total = 0;
#pragma unroll
      for (int w = 0; w < WAVES; w++) {
        const int c = s_wtot[w];
        if (w < wave) before += c;
        total += c;
      }
      const int o = base + before + incl - pc;
      // the 8 neurons of the byte, unrolled: all activation loads go out before the first store
      st v8[8];
#pragma unroll
      for (int k = 0; k < 8; k++) {
        v8[k] = DT::fromf(0.f);
        if (p.vals_out && ((bits >> k) & 1u))
          v8[k] = __hip_atomic_load(&aall[byte * 8 + k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
#pragma unroll
      for (int k = 0; k < 8; k++) {
        if ((bits >> k) & 1u) {
          const int r = o + __popc(bits & ((1u << k) - 1u));
          p.idx_out[r] = byte * 8 + k;
          if (p.vals_out) ((st*)p.vals_out)[r] = v8[k];
        }
      }
      base += total;
      __syncthreads();
    }
    if (threadIdx.x == 0) {
      *p.count_out = base;
      __hip_atomic_store(p.arrive, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

}  // namespace cats
