// Whole CATS MLP in one streaming launch plus a small reduction launch, for 1 or 2 batch rows.
//
//   mlp_fused_kernel   One persistent workgroup of 16 waves per CU owns a contiguous range of neurons.  Its "row
//                      waves" (twelve at one batch row, eight at two) take the range's neurons one at a time (LDS
//                      ticket): gate row -> SiLU -> threshold, and
//                      for an active neuron the matching W_up row -> z.  The result of every neuron is published in an
//                      LDS slot (dead, or live with its z).  The other "down waves" own an equal part of the output columns
//                      each; they walk the slots in neuron order and, for every live one, stream their part of that
//                      neuron's W_down^T row into fp32 accumulators.  Nothing crosses a workgroup boundary while the
//                      weights stream: no mask or z round trip through memory, no arrival counters, no second launch
//                      ramp between the up and the down pass.  Each workgroup ends by storing its (nb, H) partial sums.
//   reduce_partials_kernel  adds the per-workgroup partials in workgroup order, rounds to the storage type, optionally
//                      adds the residual, writes y, and totals the per-workgroup active counts.
//
// Summation order is fixed (neurons ascending inside a workgroup, workgroups ascending in the reduction), so y is
// bitwise reproducible run to run.  The two kernels are ordered by the stream, which is the only cross-workgroup
// synchronisation there is.
//
// Inside the workgroup the producer / consumer hand-off runs through LDS: a row wave writes z, a release fence, then
// the slot state (relaxed workgroup-scope atomic); a down wave reads the state (relaxed atomic), an acquire fence,
// then z.  Both fences name the LDS address space only, so they cost an s_waitcnt lgkmcnt(0) and never wait for the
// weight loads in flight.  Down waves poll with s_sleep; all waves of a workgroup are resident together, so the
// producers always make progress.
#pragma once
#include "cats_device.h"

namespace cats {

// Experiment switch, 16 in the product build: -DCATS_FUSED_WAVES=8 builds the kernel as 512-thread workgroups (half the row
// waves, half the down waves), launched two per CU with half the neuron share each.
#ifndef CATS_FUSED_WAVES
#define CATS_FUSED_WAVES 16
#endif
constexpr int kFusedWaves = CATS_FUSED_WAVES;
static_assert(kFusedWaves == 16 || kFusedWaves == 8, "sixteen waves, or eight for the two-workgroups-per-CU experiment");
// How the 16 waves split into down waves (each owns 1 / DW of the output columns) and row waves.  A row wave keeps one
// gate row and one up row in flight and waits out a memory round trip per neuron, so at one batch row twelve of them
// keep the machine busier than eight (measured: 34.6 against 35.5 us on the Llama layer); at two batch rows the down
// waves carry twice the arithmetic per fetched row and four of them fall behind (45.6 against 42.6 us).
constexpr int fused_down_waves(int batch_template) { return (batch_template == 1 ? 4 : 8) * kFusedWaves / 16; }
constexpr int kFusedThreads = kFusedWaves * kWave;
constexpr int kFusedCB = 8;             // 64-lane chunks (of 16 bytes per lane) per block of row loads
constexpr int kFusedMaxKV = 4;          // a down wave covers KV * 64 vectors of a row: rows of up to 4 * DW * 64 vectors
// Experiment switch, off in the product build: -DCATS_FUSED_POOL=1 compiles the neuron pool described at the kernel
// (dynamic balancing between the workgroups of a group).  Measured slower than fixed shares on the MI355X, kept so the
// measurement can be repeated.
#ifndef CATS_FUSED_POOL
#define CATS_FUSED_POOL 0
#endif
constexpr bool kFusedPool = CATS_FUSED_POOL != 0;
constexpr int kFusedGroup = 8;          // consecutive workgroups (one per XCD) that share a pool of neurons
constexpr int kPoolStride = 32;         // int32 per group in the pool counter array: ticket counter at +0, finished workgroups at +16
constexpr int kArriveGroups = 8;        // groups a batch row's workgroups of the reduction launch arrive in
constexpr int kArriveStride = 32;       // int32 between arrival counters: one 128-byte line each
constexpr int kReduceCols = 32;         // fp32 columns per workgroup of the reduction kernel
constexpr int kReduceLanes = 32;        // ranges of partials summed side by side per column

// Pending: not decided yet.  Dead: no batch row keeps the neuron.  Announced: some row keeps it, its z is still being
// computed -- enough for a down wave to send for the neuron's W_down^T row.  Live: z is in the slot.
// Dynamic LDS of mlp_fused_kernel: the staged x rows, the slot states, the slot z values, and one area per down wave in
// which it regroups its sums by column before the atomics of the y32 mode.  bt: compile-time batch, vec: elements per
// 16-byte vector, dw: down waves.
// cap: slots per workgroup (fused_slot_cap).
inline size_t fused_lds_bytes(int bt, int nch, int cap, int vec, int dw) {
  const size_t nchv = (size_t)(nch + kFusedCB - 1) / kFusedCB * kFusedCB * kWave;
  return (size_t)bt * nchv * 16 + (kFusedPool ? 2 : 1) * (size_t)((cap + 3) & ~3) * 4 + (size_t)((cap * bt + 3) & ~3) * 4 +
         (size_t)dw * kWave * vec * 4;
}
// Slots a workgroup needs: its own share (tickets start after the two fixed neurons of every row wave), every neuron of
// its group's pool, and one slot per row wave for the ticket that finds the pool empty.
inline int fused_slot_cap(int spw, int rpw, int rw, bool pooled) {
  if (!pooled) return rpw;
  return (spw > 2 * rw ? spw : 2 * rw) + kFusedGroup * (rpw - spw) + rw;
}

enum FusedSlot { kSlotPending = 0, kSlotDead = 1, kSlotAnnounced = 2, kSlotLive = 3 };


struct FusedArgs {
  const u32x4* x;        // (nb, H)
  const u32x4* wg;       // (I, H); NULL when the gate activations are given (a_in)
  const u32x4* wu;       // (I, H)
  const u32x4* wd;       // (I, H) neuron-major
  const void* a_in;      // optional (nb, I) dtype: gate activations; flags = |a| > t
  uint8_t* flag_out;     // optional (nb, I)
  float* partial;        // [grid][nb][H] fp32
  float* y32;            // optional (nb, H) fp32: the workgroup adds its sums here with atomics instead of storing `partial`
  int32_t* counts;       // [grid] live neurons per workgroup
  int32_t* pool;         // optional [groups][kPoolStride], all zero between calls: see the pool description at the kernel
  const u32x4* norm_w;   // optional (H,) RMS-norm weight applied to x while it is staged
  float norm_eps;
  int H, I, nb;
  int nch;               // 64-lane vector chunks per row: ceil(row_vecs / 64)
  int row_vecs;          // H / VEC
  int rpw;               // neurons per workgroup (its own share and its part of the group's pool)
  int spw;               // of those, the workgroup's own share; == rpw without a pool
  int cap;               // slots per workgroup
  float t;               // threshold, already rounded through dtype
#ifdef CATS_TIMING
  long long* tbuf;       // [gridDim][8] wall-clock stamps (100 MHz), development builds only
#endif
};

struct ReduceArgs {
  const float* partial;  // [G][BH]; or [G][gstride] with the BH wanted columns at the front of each, when gstride is set
  size_t gstride;        // 0 = BH
  const int32_t* counts; // [G]
  void* y_out;           // (nb, H) dtype, flattened to BH
  float* y32_acc;        // instead of y_out: (nb, H) fp32 that the sums are added to, unrounded (the fp32-accumulate contract)
  const void* residual;  // optional (nb, H) dtype; may alias y_out
  const void* bias;      // optional (H,) dtype, added in fp32 before the rounding
  int H;                 // row length of y (for the bias)
  int32_t* count_out;    // optional
  int G;                 // number of partials
  int BH;                // nb * H
  // optional second output: norm2_out (nb, H) dtype = norm2_w * rms_norm(y_out) -- the norm the next consumer of the
  // hidden state starts with.  Needs H % kReduceCols == 0 (a workgroup's columns lie in one row).
  void* norm2_out;
  const void* norm2_w;   // (H,) dtype
  float norm2_eps;
  float* ssq_part;       // [gridDim] sum of squares of every workgroup's columns
  float* fin;            // [BH] the finished columns as fp32, for the workgroup that writes norm2_out
  int32_t* arrive;       // arrival counters, zero between calls: [8 rows][kArriveGroups] then [8 rows], kArriveStride apart
};

#ifdef CATS_TIMING
#define CATS_FSTAMP(cond, slot) do { if (p.tbuf && (cond)) p.tbuf[(size_t)blockIdx.x * 8 + (slot)] = wall_clock64(); } while (0)
#else
#define CATS_FSTAMP(cond, slot) do { } while (0)
#endif

// CB chunks of one row: 64 lanes x 16 bytes each, issued back to back.  Never predicated: lanes past the end of a
// short row re-read its last vector and meet a zero in the LDS copy of x.
template <int CB, bool FULL>
__device__ __forceinline__ void fused_issue(const u32x4* __restrict__ row, int c0, int vlast, int lane, u32x4 (&wv)[CB]) {
#pragma unroll
  for (int cc = 0; cc < CB; cc++) {
    const int v = (c0 + cc) * kWave + lane;
    wv[cc] = load_stream(row + (FULL ? v : min(v, vlast)));
  }
}

template <class DT, int B, int CB>
__device__ __forceinline__ void fused_dot(const u32x4 (&wv)[CB], const u32x4* xs, int nchv, int c0, int lane, float (&acc)[B]) {
#pragma unroll
  for (int cc = 0; cc < CB; cc++) {
    const int v = (c0 + cc) * kWave + lane;
#pragma unroll
    for (int b = 0; b < B; b++) acc[b] = DT::dot(wv[cc], xs[b * nchv + v], acc[b]);
  }
}

// One batch of the down pass: RB row slots of KV vectors each.  The number of loads is fixed -- a slot without a row
// reads one cached vector, the same address in every lane -- so the compiler can count loads in flight and wait for
// exactly the older batch while the newer one stays outstanding.
template <int B, int KV, int RB>
struct DownBatch {
  int rows[RB];       // neuron index, -1 = empty slot
  int slots[RB];      // the slot the neuron was published in
  float zz[RB][B];
  int cnt;
  int unresolved;     // bit u: row u was taken while only announced, its z is still to be fetched
  u32x4 wv[RB][KV];
};

// Where the down waves read what the row waves publish.  Slots are handed out in ticket order; the first slots are the
// workgroup's own share in neuron order, those after it hold neurons taken from the group's pool.
struct FusedSlots {
  int* state;    // [cap] FusedSlot; written and read with workgroup-scope atomics
  float* z;      // [cap][B]; ordered against state by LDS-only release / acquire fences
  int* row;      // pool build only: [cap] neuron of the slot, written before the slot leaves the pending state
  int* nfinal;   // pool build only: number of slots in use; an upper bound (cap) until the last row wave has left
  int cap;
  int row0;      // neuron of slot 0 (slot i of the workgroup's own share is neuron row0 + i)
};

// Fill the batch with the next neurons that some batch row keeps, in neuron order, as far as the slots are decided.
// Announced is enough to take a neuron: its row can be sent for, and fused_resolve fetches its z later; the z of a slot
// that is already live is taken here.  Blocking: wait until at least one is there or the range is exhausted.
// Non-blocking: take what is there, possibly nothing.
// The wave looks at 64 slots per pass -- lane i reads state and z of slot head + i, ballots find the decided prefix and
// the kept slots in it -- so a pass costs one LDS round trip however many dead slots it steps over.
// n: the caller's copy of the number of slots in use, refreshed here.
// ANN false: an announced slot counts as pending (the wave holds too many registers of row data to also carry the
// bookkeeping of rows whose z is still to come).
template <int B, int KV, int RB, bool ANN>
__device__ __forceinline__ void fused_collect(DownBatch<B, KV, RB>& bt, const FusedSlots& sl, int& head, int& n, bool blocking) {
  bt.cnt = 0;
  bt.unresolved = 0;
#pragma unroll
  for (int u = 0; u < RB; u++) {
    bt.rows[u] = -1;
#pragma unroll
    for (int b = 0; b < B; b++) bt.zz[u][b] = 0.f;
  }
  const int lane = threadIdx.x & (kWave - 1);
  for (;;) {
    const int idx = head + lane;
    const bool in = idx < sl.cap;  // never read past the slot array
    // past the end counts as pending: it ends the decided prefix
    int st_ = in ? __hip_atomic_load(&sl.state[idx], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) : kSlotPending;
    if (kFusedPool) n = __builtin_amdgcn_readfirstlane(__hip_atomic_load(sl.nfinal, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP));
    if (head >= n) return;
    if (idx >= n) st_ = kSlotPending;  // slots past the last one in use may never have been written
    const uint64_t pend = __ballot(ANN ? st_ == kSlotPending : (st_ == kSlotPending || st_ == kSlotAnnounced));
    uint64_t live = __ballot(ANN ? st_ >= kSlotAnnounced : st_ == kSlotLive);
    const uint64_t hasz = ANN ? __ballot(st_ == kSlotLive) : ~0ull;
    const int ready = pend ? __builtin_ctzll(pend) : kWave;  // slots head .. head + ready - 1 are decided
    if (ready == 0) {
      if (!blocking) return;
      __builtin_amdgcn_s_sleep(1);
      continue;
    }
    // acquire side of the hand-off (LDS only): the z of every slot seen live above is read after its state
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    int zv[B];
#pragma unroll
    for (int b = 0; b < B; b++) zv[b] = in ? __builtin_bit_cast(int, sl.z[idx * B + b]) : 0;
    const int rowv = kFusedPool ? (in ? sl.row[idx] : -1) : sl.row0 + idx;
    if (ready < kWave) live &= (1ull << ready) - 1ull;
#pragma unroll
    for (int u = 0; u < RB; u++) {
      if (live) {  // uniform
        const int bit = __builtin_ctzll(live);
        live &= live - 1ull;
        bt.rows[u] = __builtin_amdgcn_readlane(rowv, bit);
        if (ANN) bt.slots[u] = head + bit;
        if (!ANN || ((hasz >> bit) & 1ull)) {
#pragma unroll
          for (int b = 0; b < B; b++) bt.zz[u][b] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(zv[b], bit));
        } else {
          bt.unresolved |= 1 << u;
        }
        bt.cnt++;
      }
    }
    head += live ? __builtin_ctzll(live) : ready;  // up to the first kept slot that did not fit, else past the decided prefix
    if (bt.cnt > 0) return;
    // only dead slots so far: keep going
  }
}

// Wait until the z of every row of the batch is in its slot, and read those that fused_collect could not.  Lane u
// watches row u.
template <int B, int KV, int RB, bool ANN>
__device__ __forceinline__ void fused_resolve(DownBatch<B, KV, RB>& bt, const FusedSlots& sl) {
  if (!ANN || bt.unresolved == 0) return;  // uniform
  const int lane = threadIdx.x & (kWave - 1);
  int myslot = -1;
#pragma unroll
  for (int u = 0; u < RB; u++)
    if (lane == u && ((bt.unresolved >> u) & 1)) myslot = bt.slots[u];
  for (;;) {
    const int st_ = myslot >= 0 ? __hip_atomic_load(&sl.state[myslot], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) : kSlotLive;
    if (__ballot(st_ != kSlotLive) == 0ull) break;
    __builtin_amdgcn_s_sleep(1);
  }
  // acquire side of the hand-off (LDS only): the z of every slot seen live above is read after its state
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
  int zv[B];
#pragma unroll
  for (int b = 0; b < B; b++) zv[b] = myslot >= 0 ? __builtin_bit_cast(int, sl.z[myslot * B + b]) : 0;
#pragma unroll
  for (int u = 0; u < RB; u++) {
    if ((bt.unresolved >> u) & 1) {  // uniform
#pragma unroll
      for (int b = 0; b < B; b++) bt.zz[u][b] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(zv[b], u));
    }
  }
  bt.unresolved = 0;
}

template <int B, int KV, int RB>
__device__ __forceinline__ void fused_down_issue(DownBatch<B, KV, RB>& bt, const u32x4* __restrict__ wd, int row_vecs, const u32x4* dummy,
                                                 const int (&vidx)[KV]) {
#pragma unroll
  for (int u = 0; u < RB; u++) {
    const bool live = bt.rows[u] >= 0;  // uniform
    const u32x4* r = live ? wd + (size_t)bt.rows[u] * row_vecs : dummy;
#pragma unroll
    for (int k = 0; k < KV; k++) bt.wv[u][k] = load_stream(r + (live ? vidx[k] : 0));
  }
}

template <class DT, int B, int KV, int RB>
__device__ __forceinline__ void fused_down_consume(const DownBatch<B, KV, RB>& bt, float (&acc)[B][KV][DT::VEC]) {
#pragma unroll
  for (int u = 0; u < RB; u++) {
    if (bt.rows[u] >= 0) {  // uniform; the multiply-adds of an empty slot are skipped, its load is not
#pragma unroll
      for (int k = 0; k < KV; k++)
#pragma unroll
        for (int b = 0; b < B; b++) DT::axpy(bt.wv[u][k], bt.zz[u][b], acc[b][k]);
    }
  }
}

template <class DT, int B, bool FULL, int KV, int DW>
__global__ __launch_bounds__(kFusedThreads) void mlp_fused_kernel(FusedArgs p) {
  typedef typename DT::st st;
  constexpr int CB = kFusedCB;
  constexpr int VEC = DT::VEC;
  constexpr int RW = kFusedWaves - DW;
  constexpr int RB = 8 / (KV * B) < 1 ? 1 : 8 / (KV * B);  // row slots per batch of a down wave; two batches are in flight
  constexpr bool ANN = true;  // down waves send for a row as soon as its neuron is known to be kept (see fused_collect)
  constexpr int kXPre = 2;  // x vectors per thread fetched ahead of the first weight block
  extern __shared__ u32x4 s_fused[];
  __shared__ int s_ticket;
  __shared__ int s_nfinal;     // slots in use; an upper bound while row waves are still taking tickets
  __shared__ int s_exited;     // row waves that have left
  __shared__ int s_exhausted;  // some row wave has found the group's pool empty
  __shared__ float s_scale[B];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nchp = (p.nch + CB - 1) / CB * CB;
  const int nchv = nchp * kWave;        // padded vectors per staged x row
  const int vlast = p.row_vecs - 1;
  // Neurons.  kFusedGroup consecutive workgroups form a group that owns kFusedGroup * rpw consecutive neurons.  Each
  // workgroup has spw of them to itself; what is left at the end of the group's range is the group's pool, handed out
  // one neuron at a time (a ticket counter in memory) to whichever row wave of the group asks first once its
  // workgroup's own share is taken.  Workgroups that got few live neurons, or a fast XCD, end up with more of the pool.
  // Without a pool (spw == rpw) this is one contiguous share per workgroup.
  const bool pooled = kFusedPool && p.pool != nullptr;
  const int grp = blockIdx.x / kFusedGroup, gi = blockIdx.x - grp * kFusedGroup;
  const int g0 = grp * kFusedGroup * p.rpw;
  const int ng = min(p.I - g0, kFusedGroup * p.rpw);             // neurons of the group (>= 1 by the launch shape)
  const int gsz = min(kFusedGroup, (int)gridDim.x - grp * kFusedGroup);  // workgroups of the group
  const int row0 = g0 + gi * p.spw;
  const int n = max(0, min(p.spw, ng - gi * p.spw));             // neurons of this workgroup's own share
  const int pool0 = g0 + gsz * p.spw;
  const int psize = max(0, ng - gsz * p.spw);                    // neurons in the pool
  int32_t* const pool_ctr = pooled ? p.pool + (size_t)grp * kPoolStride : p.counts;  // only touched when pooled

  u32x4* xs = s_fused;                                       // [B][nchv]
  const int cap4 = (p.cap + 3) & ~3;
  FusedSlots sl;
  sl.state = (int*)(s_fused + B * nchv);  // [cap]
  sl.row = sl.state + cap4;               // [cap], pool build only
  sl.z = (float*)(sl.state + (kFusedPool ? 2 : 1) * cap4);  // [cap][B]
  sl.nfinal = &s_nfinal;
  sl.cap = p.cap;
  sl.row0 = row0;
  float* tr_all = sl.z + ((p.cap * B + 3) & ~3);   // [DW][64 * VEC]: where a down wave regroups its sums by column (y32 mode)

  CATS_FSTAMP(tid == 0, 0);
  const bool is_row_wave = wave >= DW;
  const int rw = wave - DW;
  const bool gate = p.wg != nullptr;

  // Position in the workgroup's range -> neuron, or -1 past the end.
  auto neuron_of = [&](int q) -> int { return q < n ? row0 + q : -1; };

  // Staging, written out once per role so that each role's loads are counted on their own: memory returns are
  // counted in issue order, x goes out first, then (row waves) the first gate block, and only x is waited for before
  // the LDS writes and the barrier -- the weight loads stay in flight across both.
  auto stage = [&](auto&& issue_first) {
    u32x4 xpre[kXPre];
#pragma unroll
    for (int k = 0; k < kXPre; k++) {
      const int i = tid + k * kFusedThreads;
      const int b = B == 1 ? 0 : i / nchv, v = i - b * nchv;
      xpre[k] = zero4();
      if (i < B * nchv && b < p.nb && v < p.row_vecs) xpre[k] = p.x[(size_t)b * p.row_vecs + v];
    }
    issue_first();
#pragma unroll
    for (int k = 0; k < kXPre; k++) {
      const int i = tid + k * kFusedThreads;
      if (i < B * nchv) xs[i] = xpre[k];
    }
    for (int i = tid + kXPre * kFusedThreads; i < B * nchv; i += kFusedThreads) {
      const int b = i / nchv, v = i - b * nchv;
      u32x4 val = zero4();
      if (b < p.nb && v < p.row_vecs) val = p.x[(size_t)b * p.row_vecs + v];
      xs[i] = val;
    }
    // given activations: the down waves decide every slot (announced or dead) while they stage the activations.
    // Tickets start at 2 * RW: the slots between a short share and that point are never taken.
    if (gate)
      for (int i = tid; i < p.cap; i += kFusedThreads) sl.state[i] = (i >= n && i < 2 * RW) ? kSlotDead : kSlotPending;
    if (kFusedPool)
      for (int i = tid; i < n; i += kFusedThreads) sl.row[i] = row0 + i;
    // gate mode: the first two neurons of every row wave are fixed, the rest go by ticket; given activations: all by ticket
    if (tid == 0) {
      s_ticket = gate ? 2 * RW : 0;
      s_nfinal = (gate && pooled) ? p.cap : n;
      s_exited = 0;
      s_exhausted = 0;
    }
    __syncthreads();
    if (p.norm_w) {
      // RMS norm of each batch row, in place in LDS: one wave adds a row's squares (fixed order), everyone rescales.
      for (int b = wave; b < B; b += kFusedWaves) {
        float ss = 0.f;
        for (int v = lane; v < p.row_vecs; v += kWave) ss = vec_sumsq<DT>(xs[b * nchv + v], ss);
        ss = wave_sum(ss);
        if (lane == 0) s_scale[b] = rsqrtf(ss / (float)p.H + p.norm_eps);
      }
      __syncthreads();
      for (int i = tid; i < B * nchv; i += kFusedThreads) {
        const int b = B == 1 ? 0 : i / nchv, v = i - b * nchv;
        if (b < p.nb && v < p.row_vecs) xs[i] = vec_norm_apply<DT>(xs[i], s_scale[b], p.norm_w[v]);
      }
      __syncthreads();
    }
    CATS_FSTAMP(tid == 0, 1);
  };

  if (is_row_wave && !gate) {
    // ---- row waves, gate activations given: the down waves have put them into the z slots while x was staged (and
    // marked every slot announced or dead), so a wave knows whether a neuron is live from one LDS read.  It walks its
    // tickets and keeps the up rows of two live neurons (in blocks of CB chunks) in flight: the block of the next unit goes out
    // before the current one is multiplied, both buffers always take a full block of loads (x, cached, when there is
    // nothing left) so the wait for the older one is a fixed count.
    stage([] {});
    const int nblk = nchp / CB;
    int irow = -1, iblk = 0;  // the neuron whose blocks are being issued
    float ia[B];
    bool iact[B];
    auto next_live = [&]() -> int {
      for (;;) {
        int q = 0;
        if (lane == 0) q = __hip_atomic_fetch_add(&s_ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        q = __builtin_amdgcn_readfirstlane(q);
        if (q >= n) return -1;
        bool any = false;
#pragma unroll
        for (int b = 0; b < B; b++) {
          ia[b] = sl.z[q * B + b];
          iact[b] = b < p.nb && fabsf(ia[b]) > p.t;
          any = any || iact[b];
        }
        any = __builtin_amdgcn_readfirstlane((int)any) != 0;
        if (lane == 0 && p.flag_out) {
#pragma unroll
          for (int b = 0; b < B; b++)
            if (b < p.nb) p.flag_out[(size_t)b * p.I + row0 + q] = iact[b] ? 1 : 0;
        }
        if (any) return row0 + q;  // a dead neuron's slot already says so
      }
    };
    // one unit = one block of one live neuron's up row; row < 0 = nothing left (the loads still go out, to x)
    auto issue_next = [&](u32x4 (&buf)[CB], int& urow, int& ublk, float (&ua)[B], bool (&uact)[B]) {
      if (irow < 0 || iblk == nblk) {
        irow = next_live();
        iblk = 0;
      }
      urow = irow;
      ublk = irow >= 0 ? iblk++ : 0;
#pragma unroll
      for (int b = 0; b < B; b++) {
        ua[b] = ia[b];
        uact[b] = iact[b];
      }
      const u32x4* src = urow >= 0 ? p.wu + (size_t)urow * p.row_vecs : p.x;
      fused_issue<CB, FULL>(src, ublk * CB, vlast, lane, buf);
    };
    float u[B];
    auto consume = [&](const u32x4 (&buf)[CB], int urow, int ublk, const float (&ua)[B], const bool (&uact)[B]) {
      if (urow < 0) return;  // wave-uniform
      if (ublk == 0) {
#pragma unroll
        for (int b = 0; b < B; b++) u[b] = 0.f;
      }
      fused_dot<DT, B, CB>(buf, xs, nchv, ublk * CB, lane, u);
      if (ublk != nblk - 1) return;
      float z[B];
#pragma unroll
      for (int b = 0; b < B; b++) {
        const float ub = wave_sum(u[b]);
        z[b] = uact[b] ? DT::rnd(ua[b] * DT::rnd(ub)) : 0.f;
      }
      if (lane == 0) {
        const int slot = urow - row0;
#pragma unroll
        for (int b = 0; b < B; b++) sl.z[slot * B + b] = z[b];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __hip_atomic_store(&sl.state[slot], kSlotLive, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
    };
    u32x4 bufa[CB], bufb[CB];
    int ra, ka, rb, kb;
    float aa[B], ab[B];
    bool ca[B], cb[B];
    issue_next(bufa, ra, ka, aa, ca);
    for (;;) {
      issue_next(bufb, rb, kb, ab, cb);
      consume(bufa, ra, ka, aa, ca);
      if (rb < 0) break;
      issue_next(bufa, ra, ka, aa, ca);
      consume(bufb, rb, kb, ab, cb);
      if (ra < 0) break;
    }
#ifdef CATS_TIMING
    if (p.tbuf && lane == 0) atomicMax((unsigned long long*)&p.tbuf[(size_t)blockIdx.x * 8 + 2], (unsigned long long)wall_clock64());
#endif
    return;
  }
  if (is_row_wave) {
    // ---- row waves: gate -> decision -> up -> publish ------------------------------------------------------------
    // A wave holds its current neuron, the next one (whose first gate block it prefetches) and the ticket after that.
    // A ticket past the workgroup's own share is exchanged for a neuron of the group's pool; the request to the pool's
    // counter in memory goes out with the ticket and has a whole neuron's time to come back.
    int cur = neuron_of(rw), curslot = rw;
    int nxt = neuron_of(rw + RW), nxtslot = rw + RW;
    bool last_ticket = false;  // this wave has taken its last ticket
    u32x4 wc[CB];
    stage([&] {
      const u32x4* src = cur >= 0 ? p.wg + (size_t)cur * p.row_vecs : p.x;
      fused_issue<CB, FULL>(src, 0, vlast, lane, wc);
    });
    const int nblk = nchp / CB;
    while (cur >= 0) {
      int pend = -1, pticket = 0;
      bool ask_pool = false;
      if (!last_ticket) {
        int gone = 0;
        if (lane == 0) {
          pend = __hip_atomic_fetch_add(&s_ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          gone = __hip_atomic_load(&s_exhausted, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
        pend = __builtin_amdgcn_readfirstlane(pend);
        ask_pool = pooled && pend >= n && __builtin_amdgcn_readfirstlane(gone) == 0;
        if (ask_pool && lane == 0) pticket = __hip_atomic_fetch_add(pool_ctr, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      const int row = cur;
      float a[B];
      bool act[B];
      bool any = false;
      {
        float g[B];
#pragma unroll
        for (int b = 0; b < B; b++) g[b] = 0.f;
        for (int blk = 0; blk < nblk; blk++) {
          // next block of this row, or the first block of the next row this wave will take (past the end: x, cached)
          const bool more = blk + 1 < nblk;
          const u32x4* src = more ? p.wg + (size_t)row * p.row_vecs : (nxt >= 0 ? p.wg + (size_t)nxt * p.row_vecs : p.x);
          u32x4 wn[CB];
          fused_issue<CB, FULL>(src, more ? (blk + 1) * CB : 0, vlast, lane, wn);
          fused_dot<DT, B, CB>(wc, xs, nchv, blk * CB, lane, g);
#pragma unroll
          for (int cc = 0; cc < CB; cc++) wc[cc] = wn[cc];
        }
#pragma unroll
        for (int b = 0; b < B; b++) {
          const float gr = DT::rnd(wave_sum(g[b]));
          a[b] = DT::rnd(gr / (1.f + expf(-gr)));
          act[b] = b < p.nb && fabsf(a[b]) > p.t;
          any = any || act[b];
        }
      }
      float z[B];
#pragma unroll
      for (int b = 0; b < B; b++) z[b] = 0.f;
      if (any) {  // wave-uniform
        // the down waves may send for this neuron's W_down^T row now: it travels while the W_up row does
        if (lane == 0) __hip_atomic_store(&sl.state[curslot], kSlotAnnounced, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        float u[B];
#pragma unroll
        for (int b = 0; b < B; b++) u[b] = 0.f;
        const u32x4* ur = p.wu + (size_t)row * p.row_vecs;
        for (int blk = 0; blk < nblk; blk++) {
          u32x4 wu[CB];
          fused_issue<CB, FULL>(ur, blk * CB, vlast, lane, wu);
          fused_dot<DT, B, CB>(wu, xs, nchv, blk * CB, lane, u);
        }
#pragma unroll
        for (int b = 0; b < B; b++) {
          const float ub = wave_sum(u[b]);
          z[b] = act[b] ? DT::rnd(a[b] * DT::rnd(ub)) : 0.f;
        }
      }
      if (lane == 0) {
        if (p.flag_out) {
#pragma unroll
          for (int b = 0; b < B; b++)
            if (b < p.nb) p.flag_out[(size_t)b * p.I + row] = act[b] ? 1 : 0;
        }
        const int slot = curslot;
#pragma unroll
        for (int b = 0; b < B; b++) sl.z[slot * B + b] = z[b];
        // release side (LDS only, so the gate rows in flight are not waited for): z is in LDS before the state says so
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __hip_atomic_store(&sl.state[slot], any ? kSlotLive : kSlotDead, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
      cur = nxt;
      curslot = nxtslot;
      // what the ticket taken at the top of this pass of the loop is worth
      nxt = -1;
      nxtslot = pend;
      if (pend >= 0) {  // wave-uniform
        if (pend < n) {
          nxt = row0 + pend;
        } else {
          last_ticket = true;  // unless the pool gives a neuron
          if (ask_pool) {
            const int g = __builtin_amdgcn_readfirstlane(pticket);
            if (g < psize) {
              nxt = pool0 + g;
              last_ticket = false;
            }
          }
          if (pooled && lane == 0) {
            // the slot is taken either way: it gets the pool's neuron (written before any state that lets a down wave
            // look at it: same wave, LDS keeps a wave's accesses in order), or it is dead
            if (nxt >= 0) {
              sl.row[pend] = nxt;
            } else {
              __hip_atomic_store(&sl.state[pend], kSlotDead, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
              __hip_atomic_store(&s_exhausted, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
          }
        }
      }
    }
#ifdef CATS_TIMING
    if (p.tbuf && lane == 0) atomicMax((unsigned long long*)&p.tbuf[(size_t)blockIdx.x * 8 + 2], (unsigned long long)wall_clock64());
#endif
    if (pooled && lane == 0) {
      // The last row wave to leave knows how many slots were handed out: no ticket is taken after this point.  It also
      // reports the workgroup to its group; the last workgroup of the group to do so puts both counters back to zero
      // for the next call (every ticket of this call has been taken by then).
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
      if (__hip_atomic_fetch_add(&s_exited, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) == RW - 1) {
        const int used = __hip_atomic_load(&s_ticket, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        __hip_atomic_store(&s_nfinal, used, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        if (__hip_atomic_fetch_add(pool_ctr + 16, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == gsz - 1) {
          __hip_atomic_store(pool_ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(pool_ctr + 16, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
    return;
  }

  // ---- down waves: walk the slots in neuron order, stream this wave's columns of every live neuron ----------------
  stage([&] {
    if (!gate) {
      // given activations: (nb, I) in dtype -> the z slots of this workgroup's neurons, as fp32 (exact); the row waves read
      // them from there and overwrite them with z
      const st* ain = (const st*)p.a_in;
      for (int q = tid; q < n; q += DW * kWave) {
        bool any = false;
#pragma unroll
        for (int b = 0; b < B; b++) {
          const float av = b < p.nb ? DT::tof(ain[(size_t)b * p.I + row0 + q]) : 0.f;
          sl.z[q * B + b] = av;
          any = any || (b < p.nb && fabsf(av) > p.t);
        }
        sl.state[q] = any ? kSlotAnnounced : kSlotDead;  // ordered before any reader by the staging barrier
      }
    }
  });
  const int d = wave;
  int vidx[KV];
#pragma unroll
  for (int k = 0; k < KV; k++) vidx[k] = min((k * DW + d) * kWave + lane, vlast);
  float acc[B][KV][VEC];
#pragma unroll
  for (int b = 0; b < B; b++)
#pragma unroll
    for (int k = 0; k < KV; k++)
#pragma unroll
      for (int e = 0; e < VEC; e++) acc[b][k][e] = 0.f;

  int head = 0, nlive = 0;
  int nfin = kFusedPool ? p.cap : n;  // slots in use, as far as this wave knows (the pool build refreshes it in fused_collect)
  DownBatch<B, KV, RB> ba, bb;
  // TAIL: when nothing is left to send for, finish the batch in flight and leave no load behind (whatever is still
  // outstanding when the sums are written out has to be waited for first).  Worth half a microsecond on rows of up to
  // 2 * DW * 64 vectors; with four vectors per lane per row the extra exits cost registers the wave does not have
  // (spills), so there the last round issues its (cached, unused) loads like any other.
  constexpr bool TAIL = KV < 4;
  fused_collect<B, KV, RB, ANN>(ba, sl, head, nfin, true);
  fused_down_issue<B, KV, RB>(ba, p.wd, p.row_vecs, p.x, vidx);
  for (;;) {
    if (ba.cnt == 0 && head >= nfin) break;
    fused_collect<B, KV, RB, ANN>(bb, sl, head, nfin, ba.cnt == 0);
    if (TAIL && bb.cnt == 0 && head >= nfin) {
      fused_resolve<B, KV, RB, ANN>(ba, sl);
      fused_down_consume<DT, B, KV, RB>(ba, acc);
      nlive += ba.cnt;
      break;
    }
    fused_down_issue<B, KV, RB>(bb, p.wd, p.row_vecs, p.x, vidx);
    fused_resolve<B, KV, RB, ANN>(ba, sl);
    fused_down_consume<DT, B, KV, RB>(ba, acc);
    nlive += ba.cnt;
    if (!TAIL && bb.cnt == 0 && head >= nfin) break;
    fused_collect<B, KV, RB, ANN>(ba, sl, head, nfin, bb.cnt == 0);
    if (TAIL && ba.cnt == 0 && head >= nfin) {
      fused_resolve<B, KV, RB, ANN>(bb, sl);
      fused_down_consume<DT, B, KV, RB>(bb, acc);
      nlive += bb.cnt;
      break;
    }
    fused_down_issue<B, KV, RB>(ba, p.wd, p.row_vecs, p.x, vidx);
    fused_resolve<B, KV, RB, ANN>(bb, sl);
    fused_down_consume<DT, B, KV, RB>(bb, acc);
    nlive += bb.cnt;
  }
  CATS_FSTAMP(lane == 0 && d == 0, 3);

  if (p.y32) {
    // The caller's fp32 accumulator: one atomic per column per workgroup.  A lane's sums are VEC neighbouring columns;
    // regrouped through a wave-private piece of LDS every atomic instruction covers 64 neighbouring columns (two whole
    // cache lines).  The order in which a workgroup walks its column groups is rotated by its number, so the 256
    // workgroups, which finish together, do not all queue on the same lines.
    float* tr = tr_all + d * (kWave * VEC);
    const int rot = blockIdx.x;
#pragma unroll
    for (int kk = 0; kk < KV; kk++) {
#pragma unroll
      for (int b = 0; b < B; b++) {
        if (b < p.nb) {
          float4* trv = (float4*)(tr + lane * VEC);
#pragma unroll
          for (int q = 0; q < VEC / 4; q++) {
            // which of the wave's KV column blocks goes first is rotated as well (a register select, no indexing)
            float4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int k = 0; k < KV; k++)
              if (((kk + (rot / VEC)) % KV) == k) { o.x = acc[b][k][4 * q]; o.y = acc[b][k][4 * q + 1]; o.z = acc[b][k][4 * q + 2]; o.w = acc[b][k][4 * q + 3]; }
            trv[q] = o;
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
          const int k = (kk + (rot / VEC)) % KV;
          const int col0 = (k * DW + d) * kWave * VEC;
          // all LDS reads of the round first (one wait), then the atomics back to back
          float tv[VEC];
#pragma unroll
          for (int j = 0; j < VEC; j++) tv[j] = tr[((j + rot) % VEC) * kWave + lane];
#pragma unroll
          for (int j = 0; j < VEC; j++) {
            const int col = col0 + ((j + rot) % VEC) * kWave + lane;
            if (col < p.H) unsafeAtomicAdd(p.y32 + (size_t)b * p.H + col, tv[j]);
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
          __builtin_amdgcn_wave_barrier();  // the next round overwrites tr
        }
      }
    }
  } else {
    float* mypart = p.partial + (size_t)blockIdx.x * p.nb * p.H;
#pragma unroll
    for (int k = 0; k < KV; k++) {
      const int v = (k * DW + d) * kWave + lane;
      if (v < p.row_vecs) {
#pragma unroll
        for (int b = 0; b < B; b++)
          if (b < p.nb) {
            float4* dst = (float4*)(mypart + (size_t)b * p.H + (size_t)v * VEC);
#pragma unroll
            for (int q = 0; q < VEC / 4; q++) {
              float4 o = {acc[b][k][4 * q], acc[b][k][4 * q + 1], acc[b][k][4 * q + 2], acc[b][k][4 * q + 3]};
              dst[q] = o;
            }
          }
      }
    }
  }
  if (d == 0 && lane == 0) p.counts[blockIdx.x] = nlive;
  CATS_FSTAMP(lane == 0 && d == 0, 4);
#ifdef CATS_TIMING
  if (p.tbuf && lane == 0 && d == 0) p.tbuf[(size_t)blockIdx.x * 8 + 6] = nlive;
#endif
}

// y[c] = round(sum over g of partial[g][c]) (+ residual[c]);  c runs over the nb * H flattened outputs.  A workgroup of
// 256 threads owns kReduceCols columns: 8 threads x float4 across, 32 side by side over contiguous ranges of partials
// (all loads of a range in flight together), then one thread per column adds the 32 range sums in order.  (128 columns
// and 8 ranges per workgroup, four times fewer workgroups, is no faster for the 32 partials of the sparse down kernels:
// +0.8 us per call at 8 rows.)
template <class DT>
__global__ __launch_bounds__(256) void reduce_partials_kernel(ReduceArgs p) {
  typedef typename DT::st st;
  __shared__ float s_sum[kReduceLanes][kReduceCols + 4];
  const int tid = threadIdx.x;
  constexpr int kQ = kReduceCols / 4;  // threads across: one float4 each
  static_assert(kQ * kReduceLanes == 256, "one workgroup covers kReduceCols columns x kReduceLanes ranges");
  const int cq = tid % kQ, gl = tid / kQ;
  const int col = blockIdx.x * kReduceCols + cq * 4;
  const int per = (p.G + kReduceLanes - 1) / kReduceLanes;
  const int g0 = gl * per, g1 = min(p.G, g0 + per);
  const size_t gstride = p.gstride ? p.gstride : (size_t)p.BH;
  float4 s = {0.f, 0.f, 0.f, 0.f};
  if (col < p.BH && per == 1) {
    // at most one partial per thread (the 32 neuron groups of the sparse down kernels): one load, not a batch of eight
    if (g0 < g1) s = *(const float4*)(p.partial + (size_t)g0 * gstride + col);
  } else if (col < p.BH) {
    constexpr int U = 8;
    for (int g = g0; g < g1; g += U) {
      float4 t[U];
#pragma unroll
      for (int u = 0; u < U; u++) t[u] = *(const float4*)(p.partial + (size_t)min(g + u, g1 - 1) * gstride + col);
#pragma unroll
      for (int u = 0; u < U; u++)
        if (g + u < g1) { s.x += t[u].x; s.y += t[u].y; s.z += t[u].z; s.w += t[u].w; }
    }
  }
  s_sum[gl][cq * 4 + 0] = s.x;
  s_sum[gl][cq * 4 + 1] = s.y;
  s_sum[gl][cq * 4 + 2] = s.z;
  s_sum[gl][cq * 4 + 3] = s.w;
  __syncthreads();
  if (tid < kReduceCols) {
    const int c = blockIdx.x * kReduceCols + tid;
    if (c < p.BH) {
      float tot = 0.f;
#pragma unroll
      for (int l = 0; l < kReduceLanes; l++) tot += s_sum[l][tid];
      if (p.bias) tot += DT::tof(((const st*)p.bias)[c % p.H]);
      if (p.y32_acc) {
        p.y32_acc[c] += tot;  // one thread per column, nobody else touches it during the call
      } else {
        if (p.residual) tot = DT::rnd(tot) + DT::tof(((const st*)p.residual)[c]);
        ((st*)p.y_out)[c] = DT::fromf(tot);
      }
    }
  }
  if (p.norm2_out) {
    // The norm of the finished rows needs every column's square.  Each workgroup leaves its finished columns (as fp32, the
    // values as stored, i.e. rounded to the storage type) and the sum of their squares in the workspace; the workgroup
    // that finds itself the last to arrive adds the sums per row in workgroup order -- a fixed order, so the result
    // does not vary from run to run -- and writes the normalised rows.
    // What the other workgroups leave for that one is written with device-scope atomic stores (they write through to
    // the level all XCDs share) and the wave waits for them to be acknowledged before its arrival is counted; the last
    // workgroup invalidates its caches once (acquire fence) and reads with plain vector loads.  A device-scope release
    // fence in every workgroup would order plain stores the same way, but it writes back the whole L2 each time.
    __shared__ int s_last;
    __shared__ float s_scale2;
    const int wpr = p.H / kReduceCols;   // workgroups per row
    const int brow = blockIdx.x / wpr;   // the batch row this workgroup's columns belong to (H % kReduceCols == 0)
    if (tid < kWave) {
      float v = 0.f;
      const int c = blockIdx.x * kReduceCols + tid;
      if (tid < kReduceCols && c < p.BH) {
        v = DT::tof(((const st*)p.y_out)[c]);  // this thread's own store, just above
        __hip_atomic_store(&p.fin[c], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      v = wave_sum(v * v);
      if (tid == 0) __hip_atomic_store(&p.ssq_part[blockIdx.x], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __builtin_amdgcn_s_waitcnt(0);  // every store of this wave has been acknowledged
      // Arrivals are counted per batch row (the rows are finished by different workgroups, side by side) and in two
      // levels, every counter in a cache line of its own: atomics on one line take their turns (12 ns each on the
      // MI355X), so 1024 workgroups on one line would queue for 12 us.  A row's workgroups form up to kArriveGroups
      // groups; the last of a group reports the group to the row's counter.
      if (tid == 0) {
        const int gsize = (wpr + kArriveGroups - 1) / kArriveGroups;
        const int wi = blockIdx.x - brow * wpr, g = wi / gsize;
        const int members = min(gsize, wpr - g * gsize), ngroups = (wpr + gsize - 1) / gsize;
        int32_t* c1 = p.arrive + (size_t)(brow * kArriveGroups + g) * kArriveStride;
        int32_t* c2 = p.arrive + (size_t)(8 * kArriveGroups + brow) * kArriveStride;
        int last = 0;
        if (__hip_atomic_fetch_add(c1, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == members - 1) {
          __hip_atomic_store(c1, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // nobody else comes to this counter in this call
          if (__hip_atomic_fetch_add(c2, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == ngroups - 1) {
            __hip_atomic_store(c2, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last = 1;
          }
        }
        s_last = last;
      }
    }
    __syncthreads();
    if (s_last) {  // uniform
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
      if (tid < kWave) {
        float ss = 0.f;
        for (int w = tid; w < wpr; w += kWave) ss += p.ssq_part[brow * wpr + w];
        ss = wave_sum(ss);
        if (tid == 0) s_scale2 = rsqrtf(ss / (float)p.H + p.norm2_eps);
      }
      __syncthreads();
      constexpr int VEC = DT::VEC;
      constexpr int U = 2;  // vectors per thread whose loads go out together
      const int row_vecs = p.H / VEC;
      const float4* f4 = (const float4*)(p.fin + (size_t)brow * p.H);
      const u32x4* w4 = (const u32x4*)p.norm2_w;
      u32x4* o4 = (u32x4*)p.norm2_out + (size_t)brow * row_vecs;
      const float sc = s_scale2;
      for (int v0 = tid; v0 < row_vecs; v0 += U * 256) {
        float4 x4[U][VEC / 4];
        u32x4 wv[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
          const int v = min(v0 + u * 256, row_vecs - 1);
#pragma unroll
          for (int q = 0; q < VEC / 4; q++) x4[u][q] = f4[(size_t)v * (VEC / 4) + q];
          wv[u] = w4[v];
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
          const int v = v0 + u * 256;
          if (v < row_vecs) {
            // the finished values are exact in the storage type: packed back, the norm is the same routine the staging
            // of x uses (weight * round(x * scale), both roundings through the storage type)
            u32x4 xv;
            if constexpr (sizeof(st) == 4) {
              xv[0] = __float_as_uint(x4[u][0].x); xv[1] = __float_as_uint(x4[u][0].y);
              xv[2] = __float_as_uint(x4[u][0].z); xv[3] = __float_as_uint(x4[u][0].w);
            } else {
#pragma unroll
              for (int q = 0; q < VEC / 4; q++) {
                xv[2 * q] = (uint32_t)DT::fromf(x4[u][q].x) | ((uint32_t)DT::fromf(x4[u][q].y) << 16);
                xv[2 * q + 1] = (uint32_t)DT::fromf(x4[u][q].z) | ((uint32_t)DT::fromf(x4[u][q].w) << 16);
              }
            }
            o4[v] = vec_norm_apply<DT>(xv, sc, wv[u]);
          }
        }
      }
    }
  }
  if (p.count_out && blockIdx.x == 0 && tid >= 64 && tid < 128) {  // second wave: total of the per-workgroup counts
    int k = 0;
    for (int g = tid - 64; g < p.G; g += kWave) k += p.counts[g];
    k = (int)wave_sum((float)k);  // far below 2^24: exact in fp32
    if (tid == 64) *p.count_out = k;
  }
}

}  // namespace cats
