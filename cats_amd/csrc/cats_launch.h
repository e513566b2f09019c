// Host-side launch interface between the C ABI (cats_api.hip) and the per-dtype kernel instantiations
// (cats_inst.hip, compiled once per dtype).
#pragma once
#include <hip/hip_runtime.h>
#include "cats_down.h"
#include "cats_down_mma.h"
#include "cats_gemv_mma.h"
#include "cats_fused.h"
#include "cats_rows.h"

namespace cats {

struct Tuning {
  int gate_variant;  // N > 0: cap the rows kernel at N workgroups per CU (dynamic-LDS floor); 0 = no cap
  int down_groups;   // 0 = default (about one workgroup per CU over all slabs)
  int down_block;    // 0 = default (1024 threads)
  int path;          // whole-MLP entry points: 0 = choose by shape, 1 = always the separate gate+up and down kernels
};

// Compute units of the current device (256 if the runtime will not say), remembered per device.
int current_device_cus();

// Launch a kernel and return the status of this launch alone.  (hipGetLastError() after a <<<>>> launch would also
// return, and clear, an error that some earlier call of the caller left behind.)  Every argument must already have
// the kernel's parameter type.
template <class K, class... A>
inline hipError_t launch_kernel(K kern, dim3 grid, dim3 block, size_t lds, hipStream_t stream, A... a) {
  void* params[] = {(void*)&a...};
  return hipLaunchKernel((const void*)kern, grid, block, params, lds, stream);
}

// Returns hipSuccess or the launch error.  `mode` is a RowsMode; bt (1, 2, 4 or 8) the compile-time batch.
template <class DT>
hipError_t launch_rows(int mode, int bt, const RowsArgs& a, hipStream_t stream);
// Whether launch_rows sends this call to the matrix-core kernel, which writes the union of the flags to a.ubytes_out
// (a byte per row) instead of a.mask_out (a bit per row).
template <class DT>
bool rows_takes_mma(int mode, int bt, const RowsArgs& a);

// Gate + up (a.w2 set) or the gate pass alone for 9..16 batch rows in one pass over the weights (matrix-core kernel with
// two groups of eight rows): whether the shape and type allow it, and the launch.
template <class DT>
bool rows_mma16_supported(const RowsArgs& a);
template <class DT>
hipError_t launch_rows_mma16(const RowsArgs& a, hipStream_t stream);

template <class DT>
hipError_t launch_down(int bt, bool zf32, const DownArgs& a, int block, hipStream_t stream);

// Sparse down on the matrix cores: 16-bit types, any number of rows up to 16, partial sums out (a.partial_out set).
// `supported` also checks that a group's list, z and operands fit in LDS.
template <class DT>
bool down_mma_supported(const DownArgs& a);
template <class DT>
hipError_t launch_down_mma(bool zf32, const DownArgs& a, hipStream_t stream);

// Single-pass MLP for 1 or 2 batch rows.  stage: 0 = both launches, 1 = streaming kernel only, 2 = reduction only.
template <class DT>
hipError_t launch_fused(int bt, int grid, int stage, const FusedArgs& a, const ReduceArgs& r, hipStream_t stream);

}  // namespace cats
