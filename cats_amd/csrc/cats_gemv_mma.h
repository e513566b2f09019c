// Dense GEMV for 3..16 batch rows of a 16-bit type on the matrix cores:  out[b, r] = x[b, :] . w[r, :]   (w row-major, N x K).
// This is the down projection of the entry point that takes W_down in the (H, I) layout of nn.Linear and has to read all
// of it; the wave-per-row kernel (rows_kernel, kGemv) is bound by its dot instructions and LDS reads from four rows on
// (65 us for the 90 MB of a Llama-7B W_down at eight rows).
//
// Tiles and operand layout are those of rows_mma_kernel (8 weight rows x 64 k per v_mfma_f32_16x16x32, eight lanes per
// 128-byte line, x in LDS in operand order, the eight waves of a workgroup split K), with these differences:
//  * the row length is arbitrary and longer than LDS holds -- at K = 11008 eight rows of x are 172 KiB -- so K is cut into
//    chunks of at most 8 waves x CS steps x 64 elements, whose x operands are double-buffered in LDS: the next chunk's x is
//    fetched into registers while the current chunk is multiplied, and stored behind it;
//  * every row is live, so there are no flags and no second matrix;
//  * nothing depends on a tile's result before the end, so a wave keeps its share of every tile's sums in MFMA
//    accumulators across all chunks, and the eight waves' shares meet in LDS once, at the end.  Between the barriers of the
//    chunk switches the waves run free, each with two (chunk, tile) items of weight loads in flight, chunk-major (a ring of
//    two register sets addressed statically: the tile loop is unrolled).  Deeper rings measure slower at both batch widths
//    (three and four items: +1 to +3 us): the CU's miss queue is full before that, and a wave that blocks at issue
//    multiplies late.
// A workgroup owns ceil(N / grid) consecutive rows (16 at N = 4096 on 256 CUs) in at most TILES tiles of eight.
// Steps past the end of a row are padding: their loads re-read the first bytes of the matrix (cached, nothing moves from
// HBM), what they brought is replaced by zeros at its use and their x operands are zero.
#pragma once
#include "cats_rows_mma.h"

namespace cats {

constexpr int kGemvMmaBufBytes = 64 * 1024;  // one x buffer: 8 waves x CS steps x 64 lanes x 16 bytes x NG groups

// dynamic LDS: two x buffers; the waves' sums, [8 waves][TILES][NG][128] floats, reuse them at the end
inline size_t gemv_mma_lds_bytes() { return 2u * kGemvMmaBufBytes; }

template <class DT, int NG, int TILES>
__global__ __launch_bounds__(kMmaThreads) void gemv_mma_kernel(RowsArgs p) {
  typedef typename DT::st st;
  static_assert(sizeof(st) == 2, "16-bit types only");
  static_assert((size_t)kMmaWaves * TILES * NG * kMmaPart * sizeof(float) <= 2u * kGemvMmaBufBytes, "the sums fit the x buffers");
  constexpr int CS = 8 / NG;                          // steps per wave and chunk
  constexpr int R = 2;                                // items in flight per wave
  constexpr int CU3 = 1;                              // chunk-loop unroll that makes every item's ring slot a constant
  static_assert((CU3 * TILES) % R == 0, "ring slots repeat with the unrolled chunk loop");
  constexpr int kXGroup = kMmaWaves * CS * kWave;     // operand vectors of one group of eight batch rows in one buffer
  extern __shared__ u32x4 xs[];                       // [2 buffers][NG][kXGroup]
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  const int rows_per = (p.N + (int)gridDim.x - 1) / (int)gridDim.x;
  const int r0 = min((int)blockIdx.x * rows_per, p.N);
  const int r1 = min(r0 + rows_per, p.N);
  const int my_tiles = (r1 - r0 + kMmaTileRows - 1) / kMmaTileRows;   // <= TILES by the launch shape

  const int steps_total = (p.K + 63) / 64;            // 64-element steps of a row; the last one may be partial
  const int per_wave = (steps_total + kMmaWaves - 1) / kMmaWaves;
  const int nchunk = (per_wave + CS - 1) / CS;
  // chunk c holds n(c) steps per wave: per_wave dealt evenly, the first chunks one more
  const int cq = per_wave / nchunk, cr = per_wave % nchunk;
  auto chunk_steps = [&](int c) { return cq + (c < cr ? 1 : 0); };
  auto chunk_first = [&](int c) { return c * cq + min(c, cr); };  // in steps per wave

  const int jl = lane & 7;
  const int piece = ((lane >> 3) & 1) * 4 + (lane >> 4);
  const int ncol = lane & 15;
  const bool keep = (lane < 32) ? (ncol < 8) : (ncol >= 8);
  const int slot = (lane >> 5) * 16 + ((lane >> 4) & 1) * 8 + (ncol & 7);

  // x operands of chunk c: slot i = (wave-major local step) * 64 + l holds batch row l % 8 (of group gb), vector
  // step * 8 + (l % 16 / 8) * 4 + l / 16 of the row, where step = 8 * chunk_first(c) + local step.  Thread tid takes slots
  // tid + k * 512.  Vectors past the end of the row and batch rows past nb are zero.
  auto fetch_x = [&](int c, u32x4 (&xv)[NG][CS]) {
    const int nc = c < nchunk ? chunk_steps(c) : 0;
    const int first = kMmaWaves * chunk_first(c < nchunk ? c : 0);
#pragma unroll
    for (int gb = 0; gb < NG; gb++)
#pragma unroll
      for (int k = 0; k < CS; k++) {
        const int i = tid + k * kMmaThreads;
        const int ls = i >> 6, l = i & 63;
        const int n = l & 15, g = l >> 4, b = gb * 8 + (n & 7), kh = n >> 3;
        const int vec = (first + ls) * 8 + kh * 4 + g;
        const bool in = ls < kMmaWaves * nc && vec < p.row_vecs && b < p.nb;
        xv[gb][k] = p.x[in ? (size_t)b * p.row_vecs + vec : 0];
      }
  };
  auto store_x = [&](int c, int buf, const u32x4 (&xv)[NG][CS]) {
    const int nc = c < nchunk ? chunk_steps(c) : 0;
    const int first = kMmaWaves * chunk_first(c < nchunk ? c : 0);
#pragma unroll
    for (int gb = 0; gb < NG; gb++)
#pragma unroll
      for (int k = 0; k < CS; k++) {
        const int i = tid + k * kMmaThreads;
        const int ls = i >> 6, l = i & 63;
        const int n = l & 15, g = l >> 4, b = gb * 8 + (n & 7), kh = n >> 3;
        const int vec = (first + ls) * 8 + kh * 4 + g;
        const bool in = ls < kMmaWaves * nc && vec < p.row_vecs && b < p.nb;
        xs[(buf * NG + gb) * kXGroup + i] = in ? xv[gb][k] : zero4();
      }
  };
  // weight loads of item (chunk c, tile t): this wave's steps are local steps wave * n(c) .. + n(c) - 1 of the chunk
  auto issue = [&](int c, int t, u32x4 (&dst)[CS]) {
    const bool item = c < nchunk && t < my_tiles;  // uniform
    const int nc = item ? chunk_steps(c) : 0;
    const int step0 = item ? kMmaWaves * chunk_first(c) + wave * nc : 0;
    const int row = r0 + t * kMmaTileRows + jl;
#pragma unroll
    for (int s = 0; s < CS; s++) {
      const int vec = (step0 + s) * 8 + piece;
      const bool mine = s < nc && row < r1 && vec < p.row_vecs;
      dst[s] = load_stream(mine ? p.w + (size_t)row * p.row_vecs + vec : p.w + piece);
    }
  };

  f32x4 acc[TILES][NG];
#pragma unroll
  for (int t = 0; t < TILES; t++)
#pragma unroll
    for (int gb = 0; gb < NG; gb++) acc[t][gb] = f32x4{0.f, 0.f, 0.f, 0.f};

  CATS_RSTAMP(0);
  u32x4 xv[NG][CS];
  fetch_x(0, xv);
  u32x4 ring[R][CS];
  __builtin_amdgcn_sched_barrier(0);
  issue(0, 0, ring[0]);   // behind x in the queue, ahead of the wait for it
  __builtin_amdgcn_sched_barrier(0);
  store_x(0, 0, xv);
  __syncthreads();
  // The other items go out after the barrier: a wave blocks at issue once the CU's miss queue is full, so everything
  // issued before the barrier delays the moment the staged x becomes usable.
#pragma unroll
  for (int i = 1; i < R; i++) {
    issue(i / TILES, i % TILES, ring[i]);
    asm volatile("" ::: "memory");  // in ring order: the counted waits below rely on it
    __builtin_amdgcn_sched_barrier(0);
  }
  CATS_RSTAMP(1);
  for (int c0 = 0; c0 < nchunk; c0 += CU3) {
#pragma unroll
   for (int cc = 0; cc < CU3; cc++) {   // chunks past the last one are empty: dummy loads, no products
    const int c = c0 + cc;
    fetch_x(c + 1, xv);  // in flight while this chunk is multiplied (past the last chunk: nothing but zeros is stored)
    const int nc = c < nchunk ? chunk_steps(c) : 0;
    const int buf = c & 1;
    const int vec0 = (kMmaWaves * chunk_first(c) + wave * nc) * 8 + piece;
#pragma unroll
    for (int t = 0; t < TILES; t++) {
      u32x4 (&w)[CS] = ring[(cc * TILES + t) % R];
      if (t < my_tiles) {  // uniform; no load is issued inside
#pragma unroll
        for (int s = 0; s < CS; s++)
          if (s < nc) {
            // what a load past the end of the row brought is replaced by zeros (x is zero there, but the bytes it
            // re-read are weights: an infinity among them must not meet that zero)
            const u32x4 wv = vec0 + s * 8 < p.row_vecs ? w[s] : zero4();
#pragma unroll
            for (int gb = 0; gb < NG; gb++)
              acc[t][gb] = Mma<DT>::run(wv, xs[(buf * NG + gb) * kXGroup + (wave * nc + s) * kWave + lane], acc[t][gb]);
          }
      }
      // refill this register set with the item R ahead (chunk-major order, TILES items per chunk)
      issue(c + (t + R) / TILES, (t + R) % TILES, w);
      asm volatile("" ::: "memory");         // keeps the loads here, a ring ahead of their use
      __builtin_amdgcn_sched_barrier(0);     // and the next item's work behind them
    }
    // the buffer written here was last read in chunk c - 1, and every wave has passed the barrier that ended it
    store_x(c + 1, (c + 1) & 1, xv);
    __syncthreads();
#ifdef CATS_TIMING
    if (c < 5) CATS_RSTAMP(2 + c);
#endif
   }
  }

  // ---- the eight waves' sums meet in LDS (the x buffers are free now), one thread per output adds them in wave order ----
  float* part = (float*)xs;  // [wave][TILES][NG][128]
#pragma unroll
  for (int t = 0; t < TILES; t++)
#pragma unroll
    for (int gb = 0; gb < NG; gb++)
      if (keep) {
        float* dst = part + ((size_t)(wave * TILES + t) * NG + gb) * kMmaPart + slot;
#pragma unroll
        for (int i = 0; i < 4; i++) dst[i * 32] = acc[t][gb][i];
      }
  __syncthreads();
  for (int o = tid; o < TILES * NG * kWave; o += kMmaThreads) {
    const int l = o & 63, gb = (o >> 6) % NG, t = (o >> 6) / NG;
    const int rj = l >> 3, rb = l & 7;
    const int row = r0 + t * kMmaTileRows + rj, b = gb * 8 + rb;
    const float* src = part + ((size_t)t * NG + gb) * kMmaPart + (rj & 3) * 32 + (rj >> 2) * 8 + rb;
    float u = 0.f;
#pragma unroll
    for (int w = 0; w < kMmaWaves; w++) u += src[(size_t)w * TILES * NG * kMmaPart] + src[(size_t)w * TILES * NG * kMmaPart + 16];
    if (t < my_tiles && row < r1 && b < p.nb) ((st*)p.zt_out)[(size_t)b * p.N + row] = DT::fromf(u);
  }
  CATS_RSTAMP(7);
}

}  // namespace cats
