// Sparse down projection for 3..16 batch rows of a 16-bit type on the matrix cores:
//   y[b, :] = sum over active j of z[b, j] * wdown_t[j, :]        (same arguments and work split as down_kernel)
//
// down_kernel spends 2 * B dot instructions per weight dword and keeps B * 8 sums per lane, which have to be folded
// across sixteen waves through LDS (256 KiB of LDS traffic at eight rows, in two passes).  Here one
// v_mfma_f32_16x16x16 multiplies sixteen weight rows by up to sixteen batch rows at once:
//   * weight operand (K x N = 16 neurons x 16 columns): lane l supplies k = 4 * (l / 16) .. + 3, n = l % 16.  The rows
//     are neuron-major in memory, so a lane loads 16 bytes (8 columns) of each of its four neurons -- every quarter wave
//     reads 256 contiguous bytes of one row per load -- and interleaves the four rows column by column in registers
//     (v_perm, as down_kernel does for its row pairs).  That gives the operands of eight MFMAs, one per column of the
//     lane's eight.
//   * z operand (M x K = 16 batch rows x 16 neurons): lane l supplies m = l % 16, k = 4 * (l / 16) .. + 3: four z values
//     of one batch row, prepared once per workgroup in LDS in list order (rows nb..15 are zero).
//   * result (M x N): lane l holds batch rows 4 * (l / 16) .. + 3 of column n = l % 16 -- 8 MFMAs x 4 registers = 32
//     accumulator registers whatever the batch, against 64 (eight rows) in down_kernel.
// A step is 16 list entries x 128 columns for one wave.  The sixteen waves of a workgroup are 4 across the slab's 512
// columns x 4 over the list (step s belongs to list wave s % 4), so only four waves' sums meet in LDS: 4 KiB per wave and
// four batch rows, one pass.  Sixteen rows cost one pass over W_down^T instead of two.
//
// Every wave runs the same number of steps with DEPTH steps of loads in flight, addressed statically (a ring of DEPTH
// register sets, the loop unrolled DEPTH times) and without control flow between issue and use -- a branch around loads
// in flight makes the compiler wait for all of them.  Steps past the end of the list are padding: their entries are -1,
// they re-read row 0 (cached) and their weights are replaced by zeros before use.
#pragma once
#include "cats_down.h"

namespace cats {

typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4d __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <class DT> struct DownMma;
template <> struct DownMma<F16> {
  static __device__ __forceinline__ f32x4d run(u32x2 z, u32x2 w, f32x4d c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, z), __builtin_bit_cast(f16x4, w), c, 0, 0, 0);
  }
};
template <> struct DownMma<BF16> {
  static __device__ __forceinline__ f32x4d run(u32x2 z, u32x2 w, f32x4d c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(i16x4, z), __builtin_bit_cast(i16x4, w), c, 0, 0, 0);
  }
};

constexpr int kDownMmaThreads = 1024;
constexpr int kDownMmaListWaves = 4;   // waves that share the list; the other factor of 16 goes across the slab
constexpr int kDownMmaStep = 16;       // list entries per step (the K of the MFMA)

// Steps each list wave runs for a list of n entries: a whole number of rounds of `depth` steps.
__host__ __device__ inline int down_mma_steps_per_wave(int n, int depth) {
  const int nsteps = (n + kDownMmaStep - 1) / kDownMmaStep;
  const int spw = (nsteps + kDownMmaListWaves - 1) / kDownMmaListWaves;
  return (spw + depth - 1) / depth * depth;
}

// Dynamic LDS: streaming phase [list, padded | z of the range | z operands]; afterwards the fold, [4][rows padded to 4][512] floats.
inline size_t down_mma_lds_bytes(int chunk, int nb, int depth) {
  const int spw = down_mma_steps_per_wave(chunk, depth);
  const size_t list = (size_t)(spw + depth) * kDownMmaListWaves * kDownMmaStep * sizeof(int);
  const size_t z = ((size_t)nb * chunk * 2 + 15) / 16 * 16;
  const size_t zop = (size_t)spw * kDownMmaListWaves * kWave * 8;
  const size_t fold = (size_t)kDownMmaListWaves * ((nb + 3) / 4 * 4) * 512 * sizeof(float);
  const size_t stream = list + z + zop;
  return (stream > fold ? stream : fold) + 64;
}

template <class DT, bool ZF32, int DEPTH>
__global__ __launch_bounds__(kDownMmaThreads) void down_mma_kernel(DownArgs p) {
  typedef typename DT::st st;
  static_assert(sizeof(st) == 2 && DT::VEC == 8, "16-bit types only");
  extern __shared__ __attribute__((aligned(16))) float s_dyn[];
  __shared__ int s_n;

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int cw = wave & 3;            // which 128 columns of the slab
  const int lw = wave >> 2;           // which steps of the list
  const int q = lane >> 4;            // k block of the MFMA operands this lane supplies / batch-row block it receives
  const int c16 = lane & 15;          // n of the weight operand, m of the z operand
  const int slab = blockIdx.x % p.nslab;
  const int group = blockIdx.x / p.nslab;
  const bool by_list = p.idx != nullptr;
  const int zcols = by_list ? p.M : p.I;
  const int j0 = group * p.chunk;
  const int j1 = min(j0 + p.chunk, zcols);

  // LDS carving (must match down_mma_lds_bytes): the list is padded for the longest possible list of this range
  const int spw_max = down_mma_steps_per_wave(p.chunk, DEPTH);
  const int list_cap = (spw_max + DEPTH) * kDownMmaListWaves * kDownMmaStep;
  int* s_list = (int*)s_dyn;
  st* s_z = (st*)(s_list + list_cap);
  u32x2* s_zop = (u32x2*)((char*)s_z + ((size_t)p.nb * p.chunk * 2 + 15) / 16 * 16);
  CATS_STAMP(0);

  // ---- 1. list of active rows and z of the range -> LDS ---------------------------------------------------------
  down_stage_list_and_z<DT, ZF32>(p, j0, j1, zcols, by_list, p.nb, s_list, s_z, &s_n);
  if (wave == 0) {
    // padding entries, up to one ring of steps past the last one that is used (its loads are issued and never read)
    const int n0 = s_n;  // written by this wave
    const int end = (down_mma_steps_per_wave(n0, DEPTH) + DEPTH) * kDownMmaListWaves * kDownMmaStep;
    for (int i = n0 + lane; i < end; i += kWave) s_list[i] = -1;
  }
  __syncthreads();
  const int n = s_n;
  const int spw = down_mma_steps_per_wave(n, DEPTH);            // steps every list wave runs
  const int nsteps = spw * kDownMmaListWaves;
  CATS_STAMP(1);

  // ---- 2. stream: DEPTH steps of loads in flight per wave; the first ring goes out before the z operands are built ----
  f32x4d acc[8];
#pragma unroll
  for (int e = 0; e < 8; e++) acc[e] = f32x4d{0.f, 0.f, 0.f, 0.f};
  // Lanes past the end of a row (H not a multiple of 512) re-read the row's last vector; their sums are dropped below.
  const int v = min(slab * kWave + cw * 16 + c16, p.row_vecs - 1);
  const u32x4* wbase = p.wd + v;
  const int4* s_list4 = (const int4*)s_list;
  u32x4 w[DEPTH][4];
#pragma unroll
  for (int d = 0; d < DEPTH; d++) {
    const int4 rows = s_list4[(lw + kDownMmaListWaves * d) * 4 + q];
    w[d][0] = load_stream(wbase + (size_t)max(rows.x, 0) * p.row_vecs);
    w[d][1] = load_stream(wbase + (size_t)max(rows.y, 0) * p.row_vecs);
    w[d][2] = load_stream(wbase + (size_t)max(rows.z, 0) * p.row_vecs);
    w[d][3] = load_stream(wbase + (size_t)max(rows.w, 0) * p.row_vecs);
    asm volatile("" ::: "memory");  // in ring order, as in the loop below: the counted waits there rely on it
    __builtin_amdgcn_sched_barrier(0);
  }
  // z operands: entry (step s, lane l) = z[b = l % 16][list entries 16 s + 4 (l / 16) .. + 3], zero past nb or n
  for (int i = tid; i < nsteps * kWave; i += blockDim.x) {
    const int s = i >> 6, l = i & 63;
    const int b = l & 15, k0 = s * kDownMmaStep + 4 * (l >> 4);
    uint32_t zz[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int k = k0 + r;
      zz[r] = 0;
      if (k < n && b < p.nb) zz[r] = s_z[b * p.chunk + (by_list ? k : s_list[k] - j0)];
    }
    u32x2 o = {zz[0] | (zz[1] << 16), zz[2] | (zz[3] << 16)};
    s_zop[i] = o;
  }
  // a barrier for LDS only: __syncthreads() would also wait for the weight loads in flight
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
  for (int t0 = 0; t0 < spw; t0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; d++) {
      const int s = lw + kDownMmaListWaves * (t0 + d);
      const u32x2 zop = s_zop[s * kWave + lane];
      const int4 nxt = s_list4[(s + kDownMmaListWaves * DEPTH) * 4 + q];   // the step that takes this register set next
      const int k0 = s * kDownMmaStep + 4 * q;
      u32x4 w0 = w[d][0], w1 = w[d][1], w2 = w[d][2], w3 = w[d][3];
      // padding entries hold whatever row 0 holds: replace by zeros, so that an infinity there cannot become a NaN
      if (k0 + 0 >= n) w0 = zero4();
      if (k0 + 1 >= n) w1 = zero4();
      if (k0 + 2 >= n) w2 = zero4();
      if (k0 + 3 >= n) w3 = zero4();
#pragma unroll
      for (int i = 0; i < 4; i++) {
        // columns 2i (low halves) and 2i + 1 (high halves) of the lane's eight, rows 0..3 of its k block
        const u32x2 lo = {__builtin_amdgcn_perm(w1[i], w0[i], 0x05040100u), __builtin_amdgcn_perm(w3[i], w2[i], 0x05040100u)};
        const u32x2 hi = {__builtin_amdgcn_perm(w1[i], w0[i], 0x07060302u), __builtin_amdgcn_perm(w3[i], w2[i], 0x07060302u)};
        acc[2 * i] = DownMma<DT>::run(zop, lo, acc[2 * i]);
        acc[2 * i + 1] = DownMma<DT>::run(zop, hi, acc[2 * i + 1]);
      }
      w[d][0] = load_stream(wbase + (size_t)max(nxt.x, 0) * p.row_vecs);
      w[d][1] = load_stream(wbase + (size_t)max(nxt.y, 0) * p.row_vecs);
      w[d][2] = load_stream(wbase + (size_t)max(nxt.z, 0) * p.row_vecs);
      w[d][3] = load_stream(wbase + (size_t)max(nxt.w, 0) * p.row_vecs);
      // keeps the four loads here, a ring ahead of their use: without it the compiler carries the row numbers round the
      // loop instead and loads each row just before it is needed
      asm volatile("" ::: "memory");
      // ... and keeps the next step's work behind them: scheduled ahead, its first use of a loaded register would wait
      // for every load in flight
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  CATS_STAMP(2);

  // ---- 3. fold the four list waves through LDS and store the workgroup's partial sums --------------------------------
  // LDS: float4 slot ((lw * nbp + b) * 128 + 2 * L + (h ^ swz)) holds columns 8 L + 4 h .. + 3 of batch row b, where
  // L = cw * 16 + c16 is the lane's place across the slab and swz = (L >> 3) & 1 swaps the two halves in every other
  // group of eight lanes, so that neither the writes (lane stride 32 bytes) nor the reads meet bank conflicts.
  const int nbp = (p.nb + 3) & ~3;
  float4* s_red4 = (float4*)s_dyn;
  __syncthreads();  // list, z and operands are dead from here on
  CATS_STAMP(4);
  if (4 * q < p.nb) {
    const int L = cw * 16 + c16;
    const int swz = (L >> 3) & 1;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const float4 v4 = {acc[4 * h][i], acc[4 * h + 1][i], acc[4 * h + 2][i], acc[4 * h + 3][i]};
        s_red4[((size_t)(lw * nbp + 4 * q + i) * 128) + 2 * L + (h ^ swz)] = v4;
      }
  }
  __syncthreads();
  for (int it = tid; it < p.nb * 128; it += blockDim.x) {
    const int b = it >> 7, r = it & 127;
    const int L = r >> 1, ps = r & 1;
    const int h = ps ^ ((L >> 3) & 1);
    float4 s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int g = 0; g < kDownMmaListWaves; g++) {
      const float4 v4 = s_red4[(size_t)(g * nbp + b) * 128 + r];
      s4.x += v4.x; s4.y += v4.y; s4.z += v4.z; s4.w += v4.w;
    }
    const int col = (slab * kWave + L) * 8 + 4 * h;
    if (col < p.H) *(float4*)&p.partial[((size_t)group * p.nb + b) * p.H + col] = s4;
  }
  CATS_STAMP(5);
  if (p.count_out && blockIdx.x == 0) {
    __syncthreads();
    down_count_mask(p, s_dyn);
  }
  CATS_STAMP(3);
}

}  // namespace cats
