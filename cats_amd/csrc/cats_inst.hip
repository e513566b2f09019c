// Kernel instantiations for one dtype.  Compiled three times (-DCATS_DT=F16 / BF16 / F32) so the
// translation units build in parallel.
#include <mutex>
#include <unordered_map>

#include "cats_launch.h"
#include "cats_rows_mma.h"

#ifndef CATS_DT
#error "compile with -DCATS_DT=F16|BF16|F32"
#endif

namespace cats {

namespace {

// Kernels that want more than 48 KiB of dynamic LDS have to say so once per process (and again only if a later
// launch wants more): remembered per kernel so that the launch path makes no runtime call besides the launch.
hipError_t ensure_dynamic_lds(const void* kern, size_t bytes) {
  if (bytes <= 48 * 1024) return hipSuccess;
  static std::mutex mu;
  static std::unordered_map<uintptr_t, size_t> granted;  // (kernel, device) -> bytes; the attribute is per device
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
  const uintptr_t key = (uintptr_t)kern * 64u + (uintptr_t)dev;
  std::lock_guard<std::mutex> lock(mu);
  auto it = granted.find(key);
  if (it != granted.end() && it->second >= bytes) return hipSuccess;
  hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e == hipSuccess) granted[key] = bytes;
  return e;
}

constexpr int kR = 2;    // rows per wave per pass
constexpr int kCB = 8;   // 64-lane chunks whose loads are issued together: 8 x 16 B per lane per row
constexpr int kDownU = 8;  // rows in flight per lane in the down kernel

// Workgroup width by batch: x is staged per workgroup, so wider batches share it across more waves.
template <int B> struct WavesFor { static constexpr int value = B <= 2 ? 4 : 8; };

template <class DT, int B, bool FULL, int MODE, bool XLDS>
hipError_t launch_rows_one(const RowsArgs& a, hipStream_t stream) {
  constexpr int WAVES = WavesFor<B>::value;
  auto kern = rows_kernel<DT, B, kR, kCB, FULL, MODE, XLDS, WAVES>;
  const int rows_per_block = WAVES * kR;
  const int grid = (a.N + rows_per_block - 1) / rows_per_block;
  size_t lds = XLDS ? (size_t)B * ((a.nch + kCB - 1) / kCB * kCB) * kWave * sizeof(u32x4) : 0;
  if ((size_t)a.lds_floor > lds) lds = (size_t)a.lds_floor;
  if (hipError_t e = ensure_dynamic_lds((const void*)kern, lds); e != hipSuccess) return e;
  return launch_kernel(kern, dim3(grid), dim3(WAVES * kWave), lds, stream, a);
}

// Matrix-core gate + up pass: one persistent workgroup per CU.
template <class DT>
struct MmaLaunch {
  static bool supported(const RowsArgs&, int = 1) { return false; }
  static bool supported_up(const RowsArgs&) { return false; }
  static bool supported_gemv(const RowsArgs&) { return false; }
  static hipError_t run(const RowsArgs&, bool, hipStream_t) { return hipErrorInvalidValue; }
  static hipError_t run_up(const RowsArgs&, hipStream_t) { return hipErrorInvalidValue; }
  static hipError_t run_gemv(const RowsArgs&, hipStream_t) { return hipErrorInvalidValue; }
  static hipError_t run16(const RowsArgs&, hipStream_t) { return hipErrorInvalidValue; }
};
template <class DT>
struct MmaLaunch16 {
  static bool supported(const RowsArgs& a, int ng = 1) {
    const int steps = rows_mma_steps(a.K);
    if (a.mask_out && !a.ubytes_out) return false;  // this kernel writes the union of the flags as bytes only
    return (steps == 4 || steps == 8) && rows_mma_lds_bytes(a.K, ng) <= 160 * 1024;
  }
  // gate + up (a.w2 set) or the gate pass alone for 9..16 batch rows in one pass over the weights
  static hipError_t run16(const RowsArgs& a, hipStream_t stream) {
    const int cus = current_device_cus();
    const bool s8 = rows_mma_steps(a.K) == 8;
    auto kern = a.w2 ? (s8 ? rows_mma_kernel<DT, 8, true, 2> : rows_mma_kernel<DT, 4, true, 2>)
                     : (s8 ? rows_mma_kernel<DT, 8, false, 2> : rows_mma_kernel<DT, 4, false, 2>);
    const size_t lds = rows_mma_lds_bytes(a.K, 2);
    if (hipError_t e = ensure_dynamic_lds((const void*)kern, lds); e != hipSuccess) return e;
    const int ntiles = (a.N + kMmaTileRows - 1) / kMmaTileRows;
    return launch_kernel(kern, dim3(ntiles < cus ? ntiles : cus), dim3(kMmaThreads), lds, stream, a);
  }
  // the up pass alone, gate activations given (kUp)
  static int up_grid(const RowsArgs& a) {
    const int cus = current_device_cus();
    const int ntiles = (a.N + kMmaTileRows - 1) / kMmaTileRows;
    return ntiles < cus ? ntiles : cus;
  }
  static int up_rows_pad(const RowsArgs& a) {
    const int grid = up_grid(a);
    return ((a.N + grid - 1) / grid + kMmaTileRows - 1) / kMmaTileRows * kMmaTileRows;
  }
  static bool supported_up(const RowsArgs& a) {
    const int ng = a.nb > 8 ? 2 : 1;
    return supported(a, ng) && a.a_in && (a.z32_out || a.zt_out) && !a.norm_w && a.nb <= 16 &&
           rows_mma_up_lds_bytes(a.K, up_rows_pad(a), ng) <= 160 * 1024;
  }
  static hipError_t run_up(const RowsArgs& a, hipStream_t stream) {
    const int ng = a.nb > 8 ? 2 : 1;
    const bool s8 = rows_mma_steps(a.K) == 8;
    auto kern = ng == 2 ? (s8 ? rows_mma_up_kernel<DT, 8, 2> : rows_mma_up_kernel<DT, 4, 2>)
                        : (s8 ? rows_mma_up_kernel<DT, 8, 1> : rows_mma_up_kernel<DT, 4, 1>);
    const size_t lds = rows_mma_up_lds_bytes(a.K, up_rows_pad(a), ng);
    if (hipError_t e = ensure_dynamic_lds((const void*)kern, lds); e != hipSuccess) return e;
    return launch_kernel(kern, dim3(up_grid(a)), dim3(kMmaThreads), lds, stream, a);
  }
  // dense GEMV out = x . w^T (kGemv): any row length, 3..16 batch rows, up to 64 rows of w per workgroup
  static bool supported_gemv(const RowsArgs& a) {
    return a.zt_out && !a.norm_w && !a.bias && !a.scale && a.nb <= 16 && a.K % DT::VEC == 0 && up_rows_pad(a) <= 8 * kMmaTileRows;
  }
  template <int NG>
  static hipError_t run_gemv_ng(const RowsArgs& a, hipStream_t stream) {
    const int tiles = up_rows_pad(a) / kMmaTileRows;
    auto kern = tiles <= 2 ? gemv_mma_kernel<DT, NG, 2> : tiles <= 4 ? gemv_mma_kernel<DT, NG, 4> : gemv_mma_kernel<DT, NG, 8>;
    const size_t lds = gemv_mma_lds_bytes();
    if (hipError_t e = ensure_dynamic_lds((const void*)kern, lds); e != hipSuccess) return e;
    return launch_kernel(kern, dim3(up_grid(a)), dim3(kMmaThreads), lds, stream, a);
  }
  static hipError_t run_gemv(const RowsArgs& a, hipStream_t stream) { return a.nb > 8 ? run_gemv_ng<2>(a, stream) : run_gemv_ng<1>(a, stream); }
  static hipError_t run(const RowsArgs& a, bool up, hipStream_t stream) {
    const int cus = current_device_cus();  // one workgroup per CU
    const bool s8 = rows_mma_steps(a.K) == 8;
    auto kern = up ? (s8 ? rows_mma_kernel<DT, 8, true> : rows_mma_kernel<DT, 4, true>)
                   : (s8 ? rows_mma_kernel<DT, 8, false> : rows_mma_kernel<DT, 4, false>);
    const size_t lds = rows_mma_lds_bytes(a.K);
    if (hipError_t e = ensure_dynamic_lds((const void*)kern, lds); e != hipSuccess) return e;
    const int ntiles = (a.N + kMmaTileRows - 1) / kMmaTileRows;
    return launch_kernel(kern, dim3(ntiles < cus ? ntiles : cus), dim3(kMmaThreads), lds, stream, a);
  }
};
template <> struct MmaLaunch<F16> : MmaLaunch16<F16> {};
template <> struct MmaLaunch<BF16> : MmaLaunch16<BF16> {};

// Whether a call goes to the matrix-core kernel.  Measured on Llama-7B shapes: at 2 batch rows the wave-per-row kernel is
// still the faster one (28.4 vs 29.4 us).  The plain gate pass goes the same way as gate + up, so a gate call and a fused
// call produce the same activations bit for bit.
template <class DT>
bool takes_mma(int mode, int bt, const RowsArgs& a) {
  if (bt < 4 || !a.mma) return false;
  if (mode == kUp) return MmaLaunch<DT>::supported_up(a);
  if (mode == kGemv) return MmaLaunch<DT>::supported_gemv(a);
  return (mode == kGateUp || mode == kGate) && MmaLaunch<DT>::supported(a);
}

template <class DT, int B>
hipError_t launch_rows_b(int mode, const RowsArgs& a, hipStream_t stream) {
  if (takes_mma<DT>(mode, B, a))
    return mode == kUp ? MmaLaunch<DT>::run_up(a, stream) : mode == kGemv ? MmaLaunch<DT>::run_gemv(a, stream) : MmaLaunch<DT>::run(a, mode == kGateUp, stream);
  const size_t lds = (size_t)B * ((a.nch + kCB - 1) / kCB * kCB) * kWave * sizeof(u32x4);
  const bool xlds = lds <= 128 * 1024;
  const bool full = xlds && (a.K % (kWave * DT::VEC * kCB) == 0);
  switch (mode) {
    case kGate:
      if (full) return launch_rows_one<DT, B, true, kGate, true>(a, stream);
      if (xlds) return launch_rows_one<DT, B, false, kGate, true>(a, stream);
      return launch_rows_one<DT, B, false, kGate, false>(a, stream);
    case kGateUp:
      if (full) return launch_rows_one<DT, B, true, kGateUp, true>(a, stream);
      if (xlds) return launch_rows_one<DT, B, false, kGateUp, true>(a, stream);
      return launch_rows_one<DT, B, false, kGateUp, false>(a, stream);
    case kUp:
      if (xlds) return launch_rows_one<DT, B, false, kUp, true>(a, stream);
      return launch_rows_one<DT, B, false, kUp, false>(a, stream);
    case kGemv:
      if (xlds) return launch_rows_one<DT, B, false, kGemv, true>(a, stream);
      return launch_rows_one<DT, B, false, kGemv, false>(a, stream);
    case kUpIndex:
      if (xlds) return launch_rows_one<DT, B, false, kUpIndex, true>(a, stream);
      return launch_rows_one<DT, B, false, kUpIndex, false>(a, stream);
  }
  return hipErrorInvalidValue;
}

template <class DT, int B, bool ZF32>
hipError_t launch_down_one(const DownArgs& a, int block, hipStream_t stream) {
  auto kern = down_kernel<DT, B, ZF32, kDownU>;
  const int nwaves = block / kWave;
  // streaming phase: index list + z of the range; fold phase (same bytes): half the waves' partial sums
  // (index list, z, and for 16-bit types the packed z pairs)
  const size_t zbytes = (size_t)B * a.chunk * sizeof(typename DT::st);
  const size_t lds_stream = (size_t)a.chunk * sizeof(int) + (zbytes + 3) / 4 * 4 + (sizeof(typename DT::st) == 2 ? zbytes + 4 * B : 0);
  const size_t lds_fold = (size_t)nwaves * (B < 4 ? B : 4) * kWave * DT::VEC * sizeof(float);  // up to four batch rows per pass
  const size_t lds = (lds_stream > lds_fold ? lds_stream : lds_fold) + 64;
  if (hipError_t e = ensure_dynamic_lds((const void*)kern, lds); e != hipSuccess) return e;
  return launch_kernel(kern, dim3(a.nslab * a.ngroup), dim3(block), lds, stream, a);
}

#ifndef CATS_DOWN_MMA_DEPTH
#define CATS_DOWN_MMA_DEPTH 2
#endif
constexpr int kDownMmaDepth = CATS_DOWN_MMA_DEPTH;  // steps of loads a wave of the matrix-core down kernel keeps in flight

template <class DT>
struct DownMmaLaunch {
  static bool supported(const DownArgs&) { return false; }
  static hipError_t run(bool, const DownArgs&, hipStream_t) { return hipErrorInvalidValue; }
};
template <class DT>
struct DownMmaLaunch16 {
  static bool supported(const DownArgs& a) {
    return a.partial_out && a.nb >= 1 && a.nb <= 16 && down_mma_lds_bytes(a.chunk, a.nb, kDownMmaDepth) <= 150 * 1024;
  }
  static hipError_t run(bool zf32, const DownArgs& a, hipStream_t stream) {
    const size_t lds = down_mma_lds_bytes(a.chunk, a.nb, kDownMmaDepth);
    auto kern = zf32 ? down_mma_kernel<DT, true, kDownMmaDepth> : down_mma_kernel<DT, false, kDownMmaDepth>;
    if (hipError_t e = ensure_dynamic_lds((const void*)kern, lds); e != hipSuccess) return e;
    return launch_kernel(kern, dim3(a.nslab * a.ngroup), dim3(kDownMmaThreads), lds, stream, a);
  }
};
template <> struct DownMmaLaunch<F16> : DownMmaLaunch16<F16> {};
template <> struct DownMmaLaunch<BF16> : DownMmaLaunch16<BF16> {};

template <class DT, int B, bool FULL, int KV, int DW>
hipError_t launch_fused_one(int grid, const FusedArgs& a, hipStream_t stream) {
  auto kern = mlp_fused_kernel<DT, B, FULL, KV, DW>;
  const size_t lds = fused_lds_bytes(B, a.nch, a.cap, DT::VEC, DW);
  if (hipError_t e = ensure_dynamic_lds((const void*)kern, lds); e != hipSuccess) return e;
  return launch_kernel(kern, dim3(grid), dim3(kFusedThreads), lds, stream, a);
}

template <class DT, int B>
hipError_t launch_fused_b(int grid, const FusedArgs& a, hipStream_t stream) {
  const bool full = a.H % (kWave * DT::VEC * kFusedCB) == 0;
  constexpr int DW = fused_down_waves(B);
  const int kv = (a.row_vecs + DW * kWave - 1) / (DW * kWave);
#define CATS_FUSED_KV(KVV)                                                                \
  if (kv <= KVV) return full ? launch_fused_one<DT, B, true, KVV, DW>(grid, a, stream)    \
                             : launch_fused_one<DT, B, false, KVV, DW>(grid, a, stream);
  CATS_FUSED_KV(1)
  CATS_FUSED_KV(2)
  CATS_FUSED_KV(4)
#undef CATS_FUSED_KV
  return hipErrorInvalidValue;
}

}  // namespace

template <>
hipError_t launch_fused<CATS_DT>(int bt, int grid, int stage, const FusedArgs& a, const ReduceArgs& r, hipStream_t stream) {
  if (stage != 2) {
    hipError_t e = bt == 1 ? launch_fused_b<CATS_DT, 1>(grid, a, stream) : launch_fused_b<CATS_DT, 2>(grid, a, stream);
    if (e != hipSuccess) return e;
  }
  if (stage != 1) {
    const int rgrid = (r.BH + kReduceCols - 1) / kReduceCols;  // BH == 0: only the count is wanted
    return launch_kernel(reduce_partials_kernel<CATS_DT>, dim3(rgrid > 0 ? rgrid : 1), dim3(256), 0, stream, r);
  }
  return hipSuccess;
}

template <>
bool rows_takes_mma<CATS_DT>(int mode, int bt, const RowsArgs& a) { return takes_mma<CATS_DT>(mode, bt, a); }

template <>
bool down_mma_supported<CATS_DT>(const DownArgs& a) { return DownMmaLaunch<CATS_DT>::supported(a); }

template <>
hipError_t launch_down_mma<CATS_DT>(bool zf32, const DownArgs& a, hipStream_t stream) { return DownMmaLaunch<CATS_DT>::run(zf32, a, stream); }

template <>
bool rows_mma16_supported<CATS_DT>(const RowsArgs& a) { return a.mma && MmaLaunch<CATS_DT>::supported(a, 2); }

template <>
hipError_t launch_rows_mma16<CATS_DT>(const RowsArgs& a, hipStream_t stream) { return MmaLaunch<CATS_DT>::run16(a, stream); }

template <>
hipError_t launch_rows<CATS_DT>(int mode, int bt, const RowsArgs& a, hipStream_t stream) {
  switch (bt) {
    case 1: return launch_rows_b<CATS_DT, 1>(mode, a, stream);
    case 2: return launch_rows_b<CATS_DT, 2>(mode, a, stream);
    case 4: return launch_rows_b<CATS_DT, 4>(mode, a, stream);
    case 8: return launch_rows_b<CATS_DT, 8>(mode, a, stream);
  }
  return hipErrorInvalidValue;
}

template <>
hipError_t launch_down<CATS_DT>(int bt, bool zf32, const DownArgs& a, int block, hipStream_t stream) {
#define CATS_DOWN_CASE(BB)                                                         \
  case BB:                                                                         \
    return zf32 ? launch_down_one<CATS_DT, BB, true>(a, block, stream)             \
                : launch_down_one<CATS_DT, BB, false>(a, block, stream);
  switch (bt) {
    CATS_DOWN_CASE(1)
    CATS_DOWN_CASE(2)
    CATS_DOWN_CASE(4)
    CATS_DOWN_CASE(8)
  }
#undef CATS_DOWN_CASE
  return hipErrorInvalidValue;
}

}  // namespace cats
