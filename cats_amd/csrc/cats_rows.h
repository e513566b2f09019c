// Row-streaming kernel: one wavefront owns R consecutive weight rows at a time, every lane issues
// 128-bit streaming loads over the row, the dot products are accumulated in fp32 and folded across the
// wave with DPP.  One template covers the four row-major passes of the CATS MLP:
//
//   kGate    a = SiLU(x . wgate[j]) ; flag = |a| > t ; optional mask bytes
//   kGateUp  the gate pass, then for rows that came out active the matching wup row:  z = a * (x . wup[j])
//   kUp      flags and a are given; fetch wup rows with any flag set:                  out = a * (x . wup[j])
//   kGemv    plain y = W x (the dense (H,I) down projection over the zero-filled intermediate)
//   kUpIndex an index list picks the weight rows:  out[b, m] = scale[m] * act(x[b] . w[idx[m]] + bias[idx[m]])
//
// x is staged once per workgroup in LDS, zero-padded to a whole number of 64-lane vectors, and read back
// as one ds_read_b128 per lane per chunk (conflict-free: consecutive lanes, consecutive 16 bytes).
#pragma once
#include <type_traits>

#include "cats_device.h"

namespace cats {

enum RowsMode { kGate = 0, kGateUp = 1, kUp = 2, kGemv = 3, kUpIndex = 4 };

struct RowsArgs {
  const u32x4* x;        // (B, K) activations (K = row length of w)
  const u32x4* w;        // (N, K) first weight: wgate (kGate, kGateUp), wup (kUp), W (kGemv)
  const u32x4* w2;       // (N, K) wup for kGateUp
  const void* a_in;      // kUp: (nb, N) gate activations in dtype
  const uint8_t* flag_in;  // kUp: (nb, N); NULL = derive the flags from a_in:  |a| > t
  void* a_out;           // kGate: (nb, N) dtype, optional
  uint8_t* flag_out;     // kGate, kGateUp: (nb, N), optional
  uint8_t* mask_out;     // kGate, kGateUp: ceil(N/8) bytes, bit j = OR over the batch of flag[b, j]; optional
  uint8_t* ubytes_out;   // the matrix-core kernel's form of mask_out: N bytes, byte j = OR over the batch of flag[b, j].  Its
                         //   workgroups own row ranges that do not end on multiples of eight, so they cannot write whole mask bytes.
  float* z32_out;        // kGateUp: (nb, N) fp32, written for rows fetched from wup only; kUp: fp32 out, all rows
  void* zt_out;          // kGateUp, kUp, kGemv: (nb, N) dtype, every row written (0 where inactive)
  // index-list mode (kUpIndex): row m of the output is weight row row_idx[m]
  const int64_t* row_idx;  // (N,) weight rows to fetch, any order, duplicates allowed; entries outside [0, w_rows) give 0
  int w_rows;              // rows of w (bounds for row_idx)
  const void* bias;        // optional (w_rows,) dtype, added to the dot product of weight row j as bias[j]
  const void* scale;       // optional (N,) dtype, multiplies entry m after the activation (compact gate activations)
  int activation;          // 0 id, 1 relu, 2 squared relu, 3 swish -- applied in fp32 before the one rounding
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

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform by construction; say so
  constexpr int kThreads = WAVES * kWave;
  constexpr int kRowsPerBlock = WAVES * R;
  static_assert(kRowsPerBlock % 8 == 0 && kRowsPerBlock <= 32, "mask bytes are assembled in one 32-bit LDS word");

  CATS_RSTAMP(0);
  const int row0 = (blockIdx.x * WAVES + wave) * R;
  int row[R];   // weight row to read
  int orow[R];  // position in the outputs
  bool on[R];
#pragma unroll
  for (int r = 0; r < R; r++) {
    orow[r] = row0 + r < p.N ? row0 + r : p.N - 1;
    row[r] = orow[r];
    on[r] = row0 + r < p.N;
    if (MODE == kUpIndex) {
      const long long j = p.row_idx[orow[r]];
      const bool ok = j >= 0 && j < (long long)p.w_rows;
      row[r] = __builtin_amdgcn_readfirstlane(ok ? (int)j : 0);
      on[r] = on[r] && __builtin_amdgcn_readfirstlane((int)ok) != 0;  // an entry outside the matrix reads nothing and yields 0
    }
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
  if (MODE != kUp && MODE != kUpIndex) rows_issue<R, CB, FULL>(p.w, row, on, 0, p, lane, wv);
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

  if (MODE == kUpIndex) {
    // every list entry is fetched; what multiplies the dot product comes from the compact scale vector (or is 1)
    const st* sc = (const st*)p.scale;
#pragma unroll
    for (int r = 0; r < R; r++) {
      any[r] = on[r];
#pragma unroll
      for (int b = 0; b < B; b++) {
        act[r][b] = on[r] && b < p.nb;
        a[r][b] = sc ? DT::tof(sc[orow[r]]) : 1.f;
      }
    }
  } else if (MODE == kUp) {
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
              if (MODE == kGate && p.a_out) ((st*)p.a_out)[(size_t)b * p.N + row[r]] = DT::fromf(a[r][b]);
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
  if (MODE == kGateUp || MODE == kUp || MODE == kUpIndex) {
    float u[R][B];
    rows_dot<DT, B, R, CB, FULL, XLDS>(MODE == kGateUp ? p.w2 : p.w, row, any, xs, p.x, p, lane, wv, false, u);
    if (lane == 0) {
#pragma unroll
      for (int r = 0; r < R; r++)
        if (row0 + r < p.N) {
#pragma unroll
          for (int b = 0; b < B; b++)
            if (b < p.nb) {
              const size_t o = (size_t)b * p.N + orow[r];
              if (MODE == kUpIndex) {
                // fp32 all the way, one rounding at the store: dot product, bias of the weight row, activation, scale
                float v = 0.f;
                if (act[r][b]) {
                  v = u[r][b];
                  if (p.bias) v += DT::tof(((const st*)p.bias)[row[r]]);
                  if (p.activation == 1) v = fmaxf(v, 0.f);
                  else if (p.activation == 2) { v = fmaxf(v, 0.f); v = v * v; }
                  else if (p.activation == 3) v = v / (1.f + expf(-v));
                  v *= a[r][b];
                }
                ((st*)p.zt_out)[o] = DT::fromf(v);
              } else {
                const float z = act[r][b] ? DT::rnd(a[r][b] * DT::rnd(u[r][b])) : 0.f;
                if (p.z32_out && (MODE == kUp || any[r])) p.z32_out[o] = z;
                if (p.zt_out) ((st*)p.zt_out)[o] = DT::fromf(z);
              }
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
        if (byte < nbytes) p.mask_out[byte] = (uint8_t)(s_maskbits >> (8 * threadIdx.x));
      }
    }
  }
}

// Mask bytes -> ascending index list, the matching activations, and the count.  Runs after the gate kernel on the same
// stream (the launch boundary orders it after every mask byte and activation).  Each workgroup takes a contiguous
// range of mask bytes; where its part of the list starts is the number of set bits before the range, which it counts
// itself from the mask (a few KiB, served from cache) -- so there is no dependence between workgroups.  Inside the range:
// one byte (8 neurons) per thread and pass, popcount, wave prefix sum, LDS prefix over the waves, bit expansion.
struct CompactArgs {
  const uint8_t* mask;   // ceil(N / 8) bytes
  const void* a;         // (N,) activations in the storage type, 16-byte aligned, readable up to a multiple of 16 bytes
  int64_t* idx_out;      // (>= count,)
  void* vals_out;        // optional (>= count,) storage type
  int32_t* count_out;
  int N;
  int bytes_per_group;   // mask bytes per workgroup
};

template <int ESZ>
__global__ __launch_bounds__(256) void compact_kernel(CompactArgs p) {
  typedef typename std::conditional<ESZ == 2, uint16_t, uint32_t>::type st;
  constexpr int WAVES = 4;
  __shared__ int s_wtot[WAVES];
  __shared__ int s_base;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int nbytes = (p.N + 7) >> 3;
  const int byte0 = blockIdx.x * p.bytes_per_group;
  const int byte1 = min(nbytes, byte0 + p.bytes_per_group);
  auto bits_of = [&](int byte) -> uint32_t {
    uint32_t bits = p.mask[byte];
    const int rem = p.N - byte * 8;
    if (rem < 8) bits &= (1u << rem) - 1u;
    return bits;
  };
  constexpr int kVecs = ESZ * 8 / 16;  // 16-byte vectors holding the 8 activations of one mask byte
  const u32x4* avec = (const u32x4*)p.a;
  const int nvec = (p.N * ESZ + 15) / 16;  // whole vectors that hold activations (the buffer is at least that long)
  // A mask byte and its 8 activations are fetched together, and the first pass's fetch goes out before anything else:
  // with the count of the bits before the range that makes one memory round trip for the usual one-pass range.
  u32x4 av[kVecs];
  uint32_t bits = 0u;
  auto fetch = [&](int byte) {
#pragma unroll
    for (int q = 0; q < kVecs; q++) {
      const int v = byte * kVecs + q;
      av[q] = (p.vals_out && byte < byte1 && v < nvec) ? avec[v] : zero4();
    }
    bits = byte < byte1 ? bits_of(byte) : 0u;
  };
  fetch(byte0 + tid);
  // set bits before this workgroup's range (the last workgroup goes on to the end and so has the total)
  const bool last_group = blockIdx.x == gridDim.x - 1;
  int before = 0;
  for (int byte = tid; byte < byte0; byte += 256) before += __popc(bits_of(byte));
  before = (int)wave_sum((float)before);  // below 2^24: exact in fp32
  if (lane == 0) s_wtot[wave] = before;
  __syncthreads();
  if (tid == 0) s_base = s_wtot[0] + s_wtot[1] + s_wtot[2] + s_wtot[3];
  __syncthreads();
  int base = s_base;
  for (int b0 = byte0; b0 < byte1; b0 += 256) {
    const int byte = b0 + tid;
    if (b0 != byte0) fetch(byte);
    const int pc = __popc(bits);
    const int incl = wave_scan_inclusive(pc, lane);
    __syncthreads();  // s_wtot of the previous pass (or of the count above) has been read
    if (lane == kWave - 1) s_wtot[wave] = incl;
    __syncthreads();
    int pre = 0, total = 0;
#pragma unroll
    for (int w = 0; w < WAVES; w++) {
      const int c = s_wtot[w];
      if (w < wave) pre += c;
      total += c;
    }
    const int o = base + pre + incl - pc;
#pragma unroll
    for (int k = 0; k < 8; k++) {
      if ((bits >> k) & 1u) {
        const int r = o + __popc(bits & ((1u << k) - 1u));
        p.idx_out[r] = byte * 8 + k;
        if (p.vals_out) {
          const uint32_t word = av[k * ESZ / 16][(k * ESZ % 16) / 4];
          ((st*)p.vals_out)[r] = ESZ == 2 ? (st)(word >> (16 * (k & 1))) : (st)word;
        }
      }
    }
    base += total;
  }
  if (last_group && tid == 0) *p.count_out = base;
}

}  // namespace cats
