// Dense GEMV for 3..16 batch rows of a 16-bit type on the matrix cores:  out[b, r] = x[b, :] . w[r, :]   (w row-major, N x K).
// This is the down projection of the entry point that takes W_down in the (H, I) layout of nn.Linear and has to read all
// of it; the wave-per-row kernel (rows_kernel, kGemv) is bound by its dot instructions and LDS reads from four rows on
// (65 us for the 90 MB of a Llama-7B W_down at eight rows).
//
// Tiles and operand layout are those of rows_mma_kernel (8 weight rows x 64 k per v_mfma_f32_16x16x32, eight lanes per
// 128-byte line, x in LDS in operand order), with two differences: the row length is arbitrary and longer than LDS holds
// -- at K = 11008 eight rows of x are 172 KiB -- so K is cut into chunks of at most 8 waves x CS steps x 64 elements,
// whose x operands are double-buffered in LDS (the next chunk's x is fetched into registers while the current chunk is
// multiplied, and stored behind its last tile); and every row is live, so there are no flags and no second matrix.
// A workgroup owns ceil(N / grid) consecutive rows (16 at N = 4096 on 256 CUs) in tiles of eight.  Work items are
// (chunk, tile) pairs, chunk-major; two items' weight loads are in flight (a ring of two register sets, items always taken
// in pairs so that the ring is addressed statically), one barrier per item (partial sums alternate between two buffers),
// and wave 0 adds every item's 8 x 8 sums onto the tile's running sums in LDS; behind the last chunk it rounds and stores.
// Steps past the end of a row are padding: their loads re-read the first bytes of the matrix (cached, nothing moves from
// HBM) and their products are skipped, their x operands are zero.
#pragma once
#include "cats_rows_mma.h"

namespace cats {

constexpr int kGemvMmaBufBytes = 64 * 1024;  // one x buffer: 8 waves x CS steps x 64 lanes x 16 bytes x NG groups

// dynamic LDS: two x buffers | two partial buffers per group | running sums [NG][rows_pad][8]
inline size_t gemv_mma_lds_bytes(int ng, int rows_pad) {
  return 2u * kGemvMmaBufBytes + (size_t)ng * 2u * kMmaWaves * kMmaPart * sizeof(float) + (size_t)ng * rows_pad * 8 * sizeof(float);
}

template <class DT, int NG>
__global__ __launch_bounds__(kMmaThreads) void gemv_mma_kernel(RowsArgs p) {
  typedef typename DT::st st;
  static_assert(sizeof(st) == 2, "16-bit types only");
  constexpr int CS = 8 / NG;                          // steps per wave and chunk
  constexpr int kXGroup = kMmaWaves * CS * kWave;     // operand vectors of one group of eight batch rows in one buffer
  constexpr int kPartGroup = kMmaWaves * kMmaPart;
  extern __shared__ u32x4 xs[];                       // [2 buffers][NG][kXGroup]
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  const int rows_per = (p.N + (int)gridDim.x - 1) / (int)gridDim.x;
  const int rows_pad = (rows_per + kMmaTileRows - 1) / kMmaTileRows * kMmaTileRows;
  const int r0 = min((int)blockIdx.x * rows_per, p.N);
  const int r1 = min(r0 + rows_per, p.N);
  const int my_tiles = (r1 - r0 + kMmaTileRows - 1) / kMmaTileRows;
  const int pairs = (my_tiles + 1) / 2;               // items of a chunk are taken two at a time
  float* part = (float*)(xs + 2 * NG * kXGroup);      // [2][NG][kPartGroup]
  float* s_sum = part + 2 * NG * kPartGroup;          // [NG][rows_pad][8]

  const int steps_total = (p.K + 63) / 64;            // 64-element steps of a row; the last one may be partial
  const int per_wave = (steps_total + kMmaWaves - 1) / kMmaWaves;
  const int nchunk = (per_wave + CS - 1) / CS;
  // chunk c holds n(c) steps per wave: per_wave dealt evenly, the first chunks one more
  auto chunk_steps = [&](int c) { return per_wave / nchunk + (c < per_wave % nchunk ? 1 : 0); };
  auto chunk_first = [&](int c) { return c * (per_wave / nchunk) + min(c, per_wave % nchunk); };  // in steps per wave

  const int jl = lane & 7;
  const int piece = ((lane >> 3) & 1) * 4 + (lane >> 4);
  const int ncol = lane & 15;
  const bool keep = (lane < 32) ? (ncol < 8) : (ncol >= 8);
  const int slot = (lane >> 5) * 16 + ((lane >> 4) & 1) * 8 + (ncol & 7);
  const int rj = lane >> 3, rb = lane & 7;

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
  auto body = [&](int c, int t, u32x4 (&ring)[CS], float* my_part) {
    const int nc = chunk_steps(c);
    const int buf = c & 1;
    // what a load past the end of the row brought is replaced by zeros here, at its use (x is zero there, but the bytes
    // it re-read are weights: an infinity among them must not meet that zero)
    const int vec0 = (kMmaWaves * chunk_first(c) + wave * nc) * 8 + piece;
    u32x4 wv[CS];
#pragma unroll
    for (int s = 0; s < CS; s++) wv[s] = vec0 + s * 8 < p.row_vecs ? ring[s] : zero4();
#pragma unroll
    for (int gb = 0; gb < NG; gb++) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < CS; s++)
        if (s < nc) acc = Mma<DT>::run(wv[s], xs[(buf * NG + gb) * kXGroup + (wave * nc + s) * kWave + lane], acc);
      if (keep) {
        float* dst = my_part + gb * kPartGroup + wave * kMmaPart + slot;
#pragma unroll
        for (int i = 0; i < 4; i++) dst[i * 32] = acc[i];
      }
    }
    // refill this register set with the item two ahead (chunk-major order, `pairs` pairs per chunk)
    const bool wrap = t + 2 >= 2 * pairs;
    issue(wrap ? c + 1 : c, wrap ? t + 2 - 2 * pairs : t + 2, ring);
    __syncthreads();
    if (wave == 0 && t < my_tiles) {
      // one thread per (row rj of the tile, batch row rb): the eight waves' sums in wave order onto the running sum
      const int row = r0 + t * kMmaTileRows + rj;
#pragma unroll
      for (int gb = 0; gb < NG; gb++) {
        const float* src = my_part + gb * kPartGroup + (rj & 3) * 32 + (rj >> 2) * 8 + rb;
        float u = 0.f;
#pragma unroll
        for (int w = 0; w < kMmaWaves; w++) u += src[w * kMmaPart] + src[w * kMmaPart + 16];
        float* sum = s_sum + ((size_t)gb * rows_pad + t * kMmaTileRows + rj) * 8 + rb;
        const float tot = c == 0 ? u : *sum + u;
        const int b = gb * 8 + rb;
        if (c + 1 < nchunk) *sum = tot;
        else if (row < r1 && b < p.nb) ((st*)p.zt_out)[(size_t)b * p.N + row] = DT::fromf(tot);
      }
    }
  };

  CATS_RSTAMP(0);
  u32x4 xv[NG][CS];
  fetch_x(0, xv);
  u32x4 w0[CS], w1[CS];
  __builtin_amdgcn_sched_barrier(0);
  issue(0, 0, w0);   // behind x in the queue, ahead of the wait for it
  issue(0, 1, w1);
  __builtin_amdgcn_sched_barrier(0);
  store_x(0, 0, xv);
  __syncthreads();
  CATS_RSTAMP(1);
  for (int c = 0; c < nchunk; c++) {
    fetch_x(c + 1, xv);  // in flight while this chunk is multiplied (past the last chunk: nothing but zeros is stored)
    for (int t = 0; t < 2 * pairs; t += 2) {
      body(c, t, w0, part);
      body(c, t + 1, w1, part + NG * kPartGroup);
    }
    // every wave is past its last product with this chunk's neighbour buffer only after the barrier of the last body
    // of the chunk before; the buffer written here was last read in chunk c - 1
    store_x(c + 1, (c + 1) & 1, xv);
    __syncthreads();
  }
  CATS_RSTAMP(7);
}

}  // namespace cats
