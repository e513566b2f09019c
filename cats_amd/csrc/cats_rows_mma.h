// Gate and fused gate + up pass for batches of 3..8 rows in 16-bit types, on the matrix cores.
//
// Why not the wave-per-row kernel: with B batch rows every 16-byte weight vector costs 4 * B v_dot2 and B / 2
// LDS reads of x per lane.  From B = 4 on, that arithmetic plus the LDS traffic takes as long as the HBM stream
// itself and the three do not overlap inside a wave.  One v_mfma_f32_16x16x32 eats 1 KiB of weights against all
// batch rows at once, with one 16-byte LDS read per lane, so the kernel goes back to being a weight stream.
//
// Tile shape.  The MFMA wants 16 "rows" x 32 k per instruction with 4 lanes per row, i.e. 64 contiguous bytes
// per weight row per load instruction -- half a cache line, which streams about 25 % slower than whole lines.
// So a tile is 8 weight rows x 64 k instead: MFMA row m holds weight row m % 8, k half m / 8, and MFMA column n
// holds batch row n % 8 with the same k half n / 8.  Eight lanes then read 128 contiguous bytes of a row.  The
// (m < 8, n < 8) and (m >= 8, n >= 8) quadrants of the result are the two halves of the dot products, the other
// two quadrants pair mismatched halves and are dropped.
//
// Work split.  One persistent workgroup per CU: x is staged once in LDS in operand order (one linear 16-byte
// read per lane per step).  A workgroup owns ceil(N / grid) consecutive rows -- the same number of weight bytes for
// every CU; dealing whole tiles instead leaves 96 of 256 workgroups with 6 tiles against 5 at N = 11008 and spreads their
// ends over 4-6 us instead of 1.3-2 (the kernel's duration is the same: the memory system is the limit) -- cut into
// tiles of eight, the last one partial (its missing rows fetch nothing).  The rows of a range do not end on multiples of eight, so the union of the flags goes out as one byte
// per row (ubytes_out) rather than as bits.  The waves of a workgroup split K.  Tiles move through a software
// pipeline, one per round:
//   round r:  MFMA on the gate rows of tile r (loaded two rounds ago) -> per-wave partial sums to LDS;
//             gate loads of tile r + 2 go out; wave 0 adds the partials in wave order, applies SiLU and the
//             threshold and publishes the tile's union bits; up loads of tile r go out for the active rows only
//             (lanes of inactive rows re-read one cached line, so no HBM bytes move for them); MFMA on the up rows of tile
//             r - 1 (loaded one round ago) -> partials -> wave 0 writes z = a * up for tile r - 1.
// So the gate rows of two tiles and the up rows of one are in flight while a fourth tile is being reduced; the
// only exposed latencies are the first gate load and the last up load.  The two load rings are addressed
// statically (the loop is unrolled by two): a register that a load in flight will write cannot be moved.
#pragma once
#include "cats_rows.h"

namespace cats {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <class DT> struct Mma;
template <> struct Mma<F16> {
  static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mma<BF16> {
  static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};

constexpr int kMmaWaves = 8;
constexpr int kMmaThreads = kMmaWaves * kWave;
constexpr int kMmaTileRows = 8;
constexpr int kMmaPart = 128;    // floats per wave in a partial buffer (the two useful quadrants)

// dynamic LDS: x operands, gate partials, up partials -- each once per group of eight batch rows (ng = 1 or 2)
inline size_t rows_mma_lds_bytes(int K, int ng = 1) {
  return (size_t)ng * ((size_t)(K / 64) * kWave * sizeof(u32x4) + 2u * kMmaWaves * kMmaPart * sizeof(float));
}
// STEPS = 64-element k steps per wave per tile; the row length must be exactly kMmaWaves * STEPS * 64 so that no
// load or MFMA sits behind a bounds check (control flow around loads in flight makes the compiler wait for them).
inline int rows_mma_steps(int K) { return K % (kMmaWaves * 64) == 0 ? K / (kMmaWaves * 64) : 0; }

// UP = false is the gate pass alone (activations, flags and union bits out; no up rows, no z).
// NG = 2 takes 9..16 batch rows in one pass over the weights: the second group of eight rows is a second x operand in
// LDS and a second MFMA on the weight registers the first one just used, so the weights are still read once.
template <class DT, int STEPS, bool UP, int NG = 1>
__global__ __launch_bounds__(kMmaThreads) void rows_mma_kernel(RowsArgs p) {
  typedef typename DT::st st;
  extern __shared__ u32x4 xs[];  // [nsteps][64] x operands, then the partial buffers
  __shared__ uint32_t s_any;

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr int kMmaSteps = STEPS;
  constexpr int nsteps = kMmaWaves * STEPS;
  constexpr int kXGroup = nsteps * kWave;             // operand vectors of one group of eight batch rows
  constexpr int kPartGroup = kMmaWaves * kMmaPart;    // partial-sum floats of one group
  float* part_g = (float*)(xs + (size_t)NG * kXGroup);
  float* part_u = part_g + NG * kPartGroup;

  const int rows_per = (p.N + (int)gridDim.x - 1) / (int)gridDim.x;
  const int r0 = min((int)blockIdx.x * rows_per, p.N);  // this workgroup's rows: [r0, r1)
  const int r1 = min(r0 + rows_per, p.N);
  const int my_tiles = (r1 - r0 + kMmaTileRows - 1) / kMmaTileRows;

  const int s0 = wave * STEPS;  // this wave's first k step
  // this lane's weight row inside a tile and its 16-byte piece of the 128-byte step
  const int jl = lane & 7;
  const int piece = ((lane >> 3) & 1) * 4 + (lane >> 4);
  // slot of this lane's accumulators in a partial buffer; the two mismatched quadrants are not stored
  const int ncol = lane & 15;
  const bool keep = (lane < 32) ? (ncol < 8) : (ncol >= 8);
  const int slot = (lane >> 5) * 16 + ((lane >> 4) & 1) * 8 + (ncol & 7);

  // Loads of tile number `it` of this workgroup, never predicated: lanes with nothing to fetch -- rows past the end of
  // the range, and with use_any the rows whose union bit is clear -- read the first bytes of the matrix over and over,
  // which stay in cache and move nothing from HBM (their sums are dropped).
  auto issue = [&](const u32x4* __restrict__ w, int it, u32x4 (&dst)[kMmaSteps], bool use_any) {
    const int row = r0 + it * kMmaTileRows + jl;
    bool mine = row < r1;
    if (use_any) mine = mine && ((s_any >> jl) & 1u);
    const u32x4* src = mine ? w + (size_t)row * p.row_vecs + piece + (size_t)s0 * 8 : w + piece;
    const int stride = mine ? 8 : 0;
#pragma unroll
    for (int c = 0; c < kMmaSteps; c++) dst[c] = load_stream(src + c * stride);
  };
  auto multiply = [&](const u32x4 (&src)[kMmaSteps], float* part) {
#pragma unroll
    for (int g = 0; g < NG; g++) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < kMmaSteps; c++) acc = Mma<DT>::run(src[c], xs[g * kXGroup + (s0 + c) * kWave + lane], acc);
      if (keep) {
        float* dst = part + g * kPartGroup + wave * kMmaPart + slot;
#pragma unroll
        for (int i = 0; i < 4; i++) dst[i * 32] = acc[i];
      }
    }
  };
  // wave 0, one thread per (row j of the tile, batch row b): adds the waves' partials in wave order
  const int rj = (lane >> 3), rb = lane & 7;
  auto reduce = [&](const float* part) -> float {
    const float* src = part + (rj & 3) * 32 + (rj >> 2) * 8 + rb;
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < kMmaWaves; w++) s += src[w * kMmaPart] + src[w * kMmaPart + 16];
    return s;
  };

  // wave 0 carries the gate results of the previous tile until its up sums arrive
  float prev_a[NG];
  bool prev_act[NG], prev_valid[NG];
#pragma unroll
  for (int g = 0; g < NG; g++) {
    prev_a[g] = 0.f;
    prev_act[g] = prev_valid[g] = false;
  }
  uint32_t prev_bits = 0u;
  int prev_row = 0;

  auto round_body = [&](int r, u32x4 (&gcur)[kMmaSteps], u32x4 (&ucur)[kMmaSteps], u32x4 (&uprev)[kMmaSteps]) {
    multiply(gcur, part_g);
    issue(p.w, r + 2, gcur, false);
    __syncthreads();
    float a[NG];
    bool act[NG], valid[NG];
#pragma unroll
    for (int g = 0; g < NG; g++) {
      a[g] = 0.f;
      act[g] = valid[g] = false;
    }
    uint32_t bits8 = 0u;
    const int row = r0 + r * kMmaTileRows + rj;
    if (wave == 0 && r < my_tiles) {
      uint64_t bal = 0ull;
#pragma unroll
      for (int g = 0; g < NG; g++) {
        const int b = g * 8 + rb;  // batch row of this thread in group g
        valid[g] = row < r1 && b < p.nb;
        const float gr = DT::rnd(reduce(part_g + g * kPartGroup));
        a[g] = DT::rnd(gr / (1.f + expf(-gr)));
        act[g] = valid[g] && fabsf(a[g]) > p.t;
        bal |= __ballot(act[g]);
        if (valid[g] && p.flag_out) p.flag_out[(size_t)b * p.N + row] = act[g] ? 1 : 0;
        if (!UP && valid[g] && p.a_out) ((st*)p.a_out)[(size_t)b * p.N + row] = DT::fromf(a[g]);
      }
#pragma unroll
      for (int j = 0; j < 8; j++) bits8 |= ((bal >> (8 * j)) & 0xffull) ? (1u << j) : 0u;
      if (lane == 0) s_any = bits8;
      if (p.ubytes_out && rb == 0 && row < r1) p.ubytes_out[row] = (uint8_t)((bits8 >> rj) & 1u);
    }
    __syncthreads();
    if (!UP) return;
    issue(p.w2, r, ucur, true);
    multiply(uprev, part_u);
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int g = 0; g < NG; g++) {
        if (r >= 1 && prev_valid[g]) {
          const float u = reduce(part_u + g * kPartGroup);
          const float z = prev_act[g] ? DT::rnd(prev_a[g] * DT::rnd(u)) : 0.f;
          const size_t o = (size_t)(g * 8 + rb) * p.N + prev_row;
          if (p.z32_out && ((prev_bits >> rj) & 1u)) p.z32_out[o] = z;
          if (p.zt_out) ((st*)p.zt_out)[o] = DT::fromf(z);
        }
        prev_a[g] = a[g]; prev_act[g] = act[g]; prev_valid[g] = valid[g];
      }
      prev_bits = bits8; prev_row = row;
    }
  };

  CATS_RSTAMP(0);
  // ---- prologue.  x is requested before the first weight load goes out, so that its read does not queue behind
  // the weight requests of the whole machine. ---------------------------------------------------------------------
  u32x4 g0[kMmaSteps], g1[kMmaSteps], u0[kMmaSteps], u1[kMmaSteps];
  {
    // nsteps * 64 operand vectors over kMmaThreads threads = STEPS per thread, all loads in flight together;
    // batch rows past nb read row 0 and store zeros
    u32x4 xv[NG][STEPS];
#pragma unroll
    for (int gb = 0; gb < NG; gb++)
#pragma unroll
      for (int k = 0; k < STEPS; k++) {
        const int i = tid + k * kMmaThreads;
        const int step = i >> 6, l = i & 63;
        const int n = l & 15, g = l >> 4, b = gb * 8 + (n & 7), kh = n >> 3;
        xv[gb][k] = p.x[(size_t)(b < p.nb ? b : 0) * p.row_vecs + step * 8 + kh * 4 + g];
      }
    // the first gate tile goes out behind x, before x is waited for: it is a memory round trip ahead when the staging is done
    __builtin_amdgcn_sched_barrier(0);
    issue(p.w, 0, g0, false);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int gb = 0; gb < NG; gb++)
#pragma unroll
      for (int k = 0; k < STEPS; k++) {
        const int i = tid + k * kMmaThreads;
        const int b = gb * 8 + (i & 7);
        xs[gb * kXGroup + i] = b < p.nb ? xv[gb][k] : zero4();
      }
#pragma unroll
    for (int c = 0; c < kMmaSteps; c++) u1[c] = zero4();  // defined before the first (unused) up product
  }
  // a barrier for LDS only: __syncthreads() would also wait for the gate loads in flight
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
  // The second gate tile goes out after the barrier: a wave blocks at issue once the CU's miss queue is full, so
  // everything issued before the barrier delays the moment the staged x becomes usable.
  issue(p.w, 1, g1, false);
  if (p.norm_w) {
    // RMS norm in place.  Operand slot i = step * 64 + l holds batch row l % 8, vector step * 8 + (l % 16 / 8) * 4 + l / 16.
    // Wave b adds the squares of batch row b (kMmaWaves == 8 rows), in a fixed order.
    __shared__ float s_scale[NG * 8];
#pragma unroll
    for (int gb = 0; gb < NG; gb++) {
      float ss = 0.f;
      for (int q = lane; q < nsteps * 8; q += kWave) ss = vec_sumsq<DT>(xs[gb * kXGroup + q * 8 + wave], ss);
      ss = wave_sum(ss);
      if (lane == 0) s_scale[gb * 8 + wave] = rsqrtf(ss / (float)p.K + p.norm_eps);
    }
    __syncthreads();
#pragma unroll
    for (int gb = 0; gb < NG; gb++)
#pragma unroll
      for (int k = 0; k < STEPS; k++) {
        const int i = tid + k * kMmaThreads;
        const int step = i >> 6, l = i & 63;
        const int n = l & 15, g = l >> 4, b = gb * 8 + (n & 7), kh = n >> 3;
        if (b < p.nb) xs[gb * kXGroup + i] = vec_norm_apply<DT>(xs[gb * kXGroup + i], s_scale[b], p.norm_w[step * 8 + kh * 4 + g]);
      }
    __syncthreads();
  }
  CATS_RSTAMP(1);

  // rounds 0 .. my_tiles: the last one only drains the up sums of the last tile
  const int last = UP ? my_tiles : my_tiles - 1;
  for (int r = 0; r <= last; r += 2) {
    round_body(r, g0, u0, u1);
    if (r + 1 <= last) round_body(r + 1, g1, u1, u0);
#ifdef CATS_TIMING
    if (r < 10) CATS_RSTAMP(2 + (r >> 1));
#endif
  }
  CATS_RSTAMP(7);
}

// The up pass alone, for callers that bring the gate activations (kUp; flags = |a| > t, or the caller's flag bytes):
//   z[b, j] = a[b, j] * (x[b] . wup[j])  where flag[b, j], else 0; rows of W_up without a flag in any batch row are not read.
// Out: the union of the flags to ubytes_out (optional); z as fp32 for the rows that were read (flags derived: the sparse
// down pass that follows reads no others) or for every row (flags given), and / or in the storage type for every row.
// Same tiles, operand layout and work split as rows_mma_kernel.  With a given, every tile's union bits are known before
// the first weight byte moves: the workgroup stages its range of a in LDS, derives the bits of all its tiles, and then
// streams W_up with two tiles in flight (a ring of two register sets, the loop unrolled by two) and one barrier per tile
// (the per-wave partial sums alternate between two buffers: wave 0 adds up tile r while the others multiply tile r + 1).
// NG = 2 takes 9..16 batch rows: a second x operand in LDS and a second MFMA on the same weight registers.
// dynamic LDS, per group of eight batch rows: x operands | two partial buffers | a of the range, [8][rows_pad] in storage
// type | its flags, [8][rows_pad] bytes; then one byte of union bits per tile
inline size_t rows_mma_up_lds_bytes(int K, int rows_pad, int ng) {
  return rows_mma_lds_bytes(K, ng) + (size_t)ng * 8 * rows_pad * 3 + (size_t)(rows_pad / 8 + 15) / 16 * 16;
}

template <class DT, int STEPS, int NG>
__global__ __launch_bounds__(kMmaThreads) void rows_mma_up_kernel(RowsArgs p) {
  typedef typename DT::st st;
  static_assert(sizeof(st) == 2, "16-bit types only");
  extern __shared__ u32x4 xs[];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr int nsteps = kMmaWaves * STEPS;
  constexpr int kXGroup = nsteps * kWave;
  constexpr int kPartGroup = kMmaWaves * kMmaPart;

  const int rows_per = (p.N + (int)gridDim.x - 1) / (int)gridDim.x;
  const int rows_pad = (rows_per + kMmaTileRows - 1) / kMmaTileRows * kMmaTileRows;
  const int r0 = min((int)blockIdx.x * rows_per, p.N);
  const int r1 = min(r0 + rows_per, p.N);
  const int my_tiles = (r1 - r0 + kMmaTileRows - 1) / kMmaTileRows;
  constexpr int NB = NG * 8;                                // batch rows the kernel is laid out for
  float* part = (float*)(xs + NG * kXGroup);                // [2][NG][kPartGroup]
  st* s_a = (st*)(part + 2 * NG * kPartGroup);              // [NB][rows_pad]
  uint8_t* s_f = (uint8_t*)(s_a + NB * rows_pad);           // [NB][rows_pad]
  uint8_t* s_bits = s_f + NB * rows_pad;                    // [rows_pad / 8]

  const int s0 = wave * STEPS;
  const int jl = lane & 7;
  const int piece = ((lane >> 3) & 1) * 4 + (lane >> 4);
  const int ncol = lane & 15;
  const bool keep = (lane < 32) ? (ncol < 8) : (ncol >= 8);
  const int slot = (lane >> 5) * 16 + ((lane >> 4) & 1) * 8 + (ncol & 7);
  const int rj = lane >> 3, rb = lane & 7;

  CATS_RSTAMP(0);
  // ---- prologue: x -> LDS in operand order (as rows_mma_kernel), a of the range -> LDS, the bits of every tile ----------
  {
    u32x4 xv[NG][STEPS];
#pragma unroll
    for (int gb = 0; gb < NG; gb++)
#pragma unroll
      for (int k = 0; k < STEPS; k++) {
        const int i = tid + k * kMmaThreads;
        const int step = i >> 6, l = i & 63;
        const int n = l & 15, g = l >> 4, b = gb * 8 + (n & 7), kh = n >> 3;
        xv[gb][k] = p.x[(size_t)(b < p.nb ? b : 0) * p.row_vecs + step * 8 + kh * 4 + g];
      }
    const st* ain = (const st*)p.a_in;
    for (int e = tid; e < NB * rows_pad; e += kMmaThreads) {
      const int b = e / rows_pad, j = e - b * rows_pad;
      const bool in = b < p.nb && r0 + j < r1;  // the padding of the range and of the batch is never flagged
      const size_t o = (size_t)b * p.N + r0 + j;
      const st av = in ? ain[o] : DT::fromf(0.f);
      s_a[e] = av;
      s_f[e] = in && (p.flag_in ? p.flag_in[o] != 0 : fabsf(DT::tof(av)) > p.t) ? 1 : 0;
    }
#pragma unroll
    for (int gb = 0; gb < NG; gb++)
#pragma unroll
      for (int k = 0; k < STEPS; k++) {
        const int i = tid + k * kMmaThreads;
        xs[gb * kXGroup + i] = gb * 8 + (i & 7) < p.nb ? xv[gb][k] : zero4();
      }
  }
  __syncthreads();
  // one thread per row of the range: any batch row flagged?  Eight neighbouring lanes make a tile's byte.
  for (int j0 = 0; j0 < rows_pad; j0 += kMmaThreads) {
    const int j = j0 + tid;
    bool any = false;
    if (j < rows_pad) {
#pragma unroll
      for (int b = 0; b < NB; b++) any = any || s_f[b * rows_pad + j] != 0;
      if (p.ubytes_out && r0 + j < r1) p.ubytes_out[r0 + j] = any ? 1 : 0;
    }
    const uint64_t bal = __ballot(any);
    if (j < rows_pad && (lane & 7) == 0) s_bits[j >> 3] = (uint8_t)((bal >> (lane & 56)) & 0xffull);
  }
  __syncthreads();
  CATS_RSTAMP(1);

  auto issue = [&](int it, u32x4 (&dst)[STEPS]) {
    const int row = r0 + it * kMmaTileRows + jl;
    const uint32_t bits = it < my_tiles ? s_bits[it] : 0u;
    const bool mine = row < r1 && ((bits >> jl) & 1u);
    const u32x4* src = mine ? p.w + (size_t)row * p.row_vecs + piece + (size_t)s0 * 8 : p.w + piece;
    const int stride = mine ? 8 : 0;
#pragma unroll
    for (int c = 0; c < STEPS; c++) dst[c] = load_stream(src + c * stride);
  };
  auto multiply = [&](const u32x4 (&src)[STEPS], float* dst_part) {
#pragma unroll
    for (int gb = 0; gb < NG; gb++) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < STEPS; c++) acc = Mma<DT>::run(src[c], xs[gb * kXGroup + (s0 + c) * kWave + lane], acc);
      if (keep) {
        float* dst = dst_part + gb * kPartGroup + wave * kMmaPart + slot;
#pragma unroll
        for (int i = 0; i < 4; i++) dst[i * 32] = acc[i];
      }
    }
  };
  auto body = [&](int r, u32x4 (&ring)[STEPS], float* my_part) {
    multiply(ring, my_part);
    issue(r + 2, ring);
    __syncthreads();
    if (wave == 0 && r < my_tiles) {
      // one thread per (row rj of the tile, batch row rb): the eight waves' partials in wave order, then z = a * up
      const int j = r * kMmaTileRows + rj;
      const int row = r0 + j;
      const bool live = (s_bits[r] >> rj) & 1u;       // the row was read
#pragma unroll
      for (int gb = 0; gb < NG; gb++) {
        const int b = gb * 8 + rb;
        const float* src = my_part + gb * kPartGroup + (rj & 3) * 32 + (rj >> 2) * 8 + rb;
        float u = 0.f;
#pragma unroll
        for (int w = 0; w < kMmaWaves; w++) u += src[w * kMmaPart] + src[w * kMmaPart + 16];
        const float a = DT::tof(s_a[b * rows_pad + j]);
        if (row < r1 && b < p.nb) {
          const float z = s_f[b * rows_pad + j] ? DT::rnd(a * DT::rnd(u)) : 0.f;  // u of a row that was not read is noise: never used
          const size_t o = (size_t)b * p.N + row;
          if (p.z32_out && (live || p.flag_in)) p.z32_out[o] = z;
          if (p.zt_out) ((st*)p.zt_out)[o] = DT::fromf(z);
        }
      }
    }
  };

  u32x4 u0[STEPS], u1[STEPS];
  issue(0, u0);
  issue(1, u1);
  // always in pairs (an odd count ends with a tile of dummy loads): a branch around the second body would leave the
  // compiler with a path on which its counted waits for the ring degrade to "wait for everything"
  for (int r = 0; r < my_tiles; r += 2) {
    body(r, u0, part);
    body(r + 1, u1, part + NG * kPartGroup);
  }
  CATS_RSTAMP(7);
}

}  // namespace cats
