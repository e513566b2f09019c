// Device-side building blocks shared by the CATS kernels: 128-bit vector type, dtype traits
// (fp16 / bf16 / fp32 storage with fp32 arithmetic), wave64 reductions and scans.
// gfx950 only: wavefronts are 64 lanes wide, DPP row operations and v_dot2 are assumed.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cats {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// Streaming (non-temporal) 128-bit load: weight rows are touched once per call, so they should not
// displace x, the mask words or the partial sums from L2.
__device__ __forceinline__ u32x4 load_stream(const u32x4* p) { return __builtin_nontemporal_load(p); }

// Bit casts of single vector lanes go through these by-value helpers: __builtin_bit_cast applied directly to a
// vector element expression (w[i]) reads lane 0 for every i with this compiler.
__device__ __forceinline__ f16x2 as_f16x2(uint32_t v) { return __builtin_bit_cast(f16x2, v); }
__device__ __forceinline__ bf16x2 as_bf16x2(uint32_t v) { return __builtin_bit_cast(bf16x2, v); }

__device__ __forceinline__ u32x4 zero4() {
  u32x4 z = {0u, 0u, 0u, 0u};
  return z;
}

// ---- dtype traits -----------------------------------------------------------------------------
// st      storage type of one element
// VEC     elements per 16-byte vector
// tof     storage -> float (exact)
// fromf   float -> storage, round to nearest even
// rnd     float -> float, rounded through the storage type
// dot     acc + sum over the VEC element pairs of two vectors, accumulated in fp32
// dot2    (16-bit types) acc + the two products of one packed pair
// axpy    acc[i] += z * w[i] for the VEC elements of one vector

struct F16 {
  typedef uint16_t st;
  static constexpr int VEC = 8;
  static __device__ __forceinline__ float tof(st b) { return (float)__builtin_bit_cast(_Float16, b); }
  static __device__ __forceinline__ st fromf(float f) { return __builtin_bit_cast(st, (_Float16)f); }
  static __device__ __forceinline__ float rnd(float f) { return (float)(_Float16)f; }
  static __device__ __forceinline__ float dot(u32x4 w, u32x4 x, float acc) {
#pragma unroll
    for (int i = 0; i < 4; i++)
      acc = __builtin_amdgcn_fdot2(as_f16x2(w[i]), as_f16x2(x[i]), acc, false);
    return acc;
  }
  static __device__ __forceinline__ float dot2(uint32_t w, uint32_t x, float acc) {
    return __builtin_amdgcn_fdot2(as_f16x2(w), as_f16x2(x), acc, false);
  }
  static __device__ __forceinline__ void axpy(u32x4 w, float z, float* acc) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const f16x2 p = as_f16x2(w[i]);
      acc[2 * i] = fmaf(z, (float)p[0], acc[2 * i]);
      acc[2 * i + 1] = fmaf(z, (float)p[1], acc[2 * i + 1]);
    }
  }
};

struct BF16 {
  typedef uint16_t st;
  static constexpr int VEC = 8;
  static __device__ __forceinline__ float tof(st b) { return __uint_as_float((uint32_t)b << 16); }
  static __device__ __forceinline__ st fromf(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (st)((u >> 16) | 0x0040u);  // quiet NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return (st)(u >> 16);
  }
  static __device__ __forceinline__ float rnd(float f) { return tof(fromf(f)); }
  static __device__ __forceinline__ float dot(u32x4 w, u32x4 x, float acc) {
#pragma unroll
    for (int i = 0; i < 4; i++)
      acc = __builtin_amdgcn_fdot2_f32_bf16(as_bf16x2(w[i]), as_bf16x2(x[i]), acc, false);
    return acc;
  }
  static __device__ __forceinline__ float dot2(uint32_t w, uint32_t x, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(as_bf16x2(w), as_bf16x2(x), acc, false);
  }
  static __device__ __forceinline__ void axpy(u32x4 w, float z, float* acc) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      acc[2 * i] = fmaf(z, __uint_as_float(w[i] << 16), acc[2 * i]);
      acc[2 * i + 1] = fmaf(z, __uint_as_float(w[i] & 0xffff0000u), acc[2 * i + 1]);
    }
  }
};

struct F32 {
  typedef float st;
  static constexpr int VEC = 4;
  static __device__ __forceinline__ float tof(st b) { return b; }
  static __device__ __forceinline__ st fromf(float f) { return f; }
  static __device__ __forceinline__ float rnd(float f) { return f; }
  static __device__ __forceinline__ float dot(u32x4 w, u32x4 x, float acc) {
#pragma unroll
    for (int i = 0; i < 4; i++) acc = fmaf(__uint_as_float(w[i]), __uint_as_float(x[i]), acc);
    return acc;
  }
  static __device__ __forceinline__ void axpy(u32x4 w, float z, float* acc) {
#pragma unroll
    for (int i = 0; i < 4; i++) acc[i] = fmaf(z, __uint_as_float(w[i]), acc[i]);
  }
};

// ---- RMS norm pieces (generic over the traits) ----------------------------------------------------
// Sum of squares of the VEC elements of one vector, in fp32.
template <class DT>
__device__ __forceinline__ float vec_sumsq(u32x4 x, float acc) {
  return DT::dot(x, x, acc);
}

// Element-wise  w * round(x * scale)  with both roundings through the storage type: the two steps of an RMS norm
// layer whose weight multiplies the already down-cast normalised activations.
template <class DT>
__device__ __forceinline__ u32x4 vec_norm_apply(u32x4 x, float scale, u32x4 w) {
  typedef typename DT::st st;
  constexpr int PER = 4 / sizeof(st);  // elements per dword
  u32x4 out;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint32_t xi = x[i], wi = w[i];  // by value: see as_f16x2
    uint32_t o = 0;
#pragma unroll
    for (int h = 0; h < PER; h++) {
      st xe, we;
      if constexpr (PER == 1) {
        xe = __builtin_bit_cast(st, xi);
        we = __builtin_bit_cast(st, wi);
      } else {
        xe = (st)(xi >> (16 * h));
        we = (st)(wi >> (16 * h));
      }
      const float xn = DT::rnd(DT::tof(xe) * scale);
      const st r = DT::fromf(DT::tof(we) * xn);
      if constexpr (PER == 1) o = __builtin_bit_cast(uint32_t, r);
      else o |= (uint32_t)r << (16 * h);
    }
    out[i] = o;
  }
  return out;
}

// ---- wave64 cross-lane helpers ------------------------------------------------------------------

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  // bound_ctrl = true: lanes whose DPP source is invalid read 0 (none are, for the controls used here).
  int o = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true);
  return v + __int_as_float(o);
}

// Sum over the 64 lanes; the result is wave-uniform.  Four DPP steps fold each row of 16 lanes
// (quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror, row_mirror), then the four row totals are
// read out with v_readlane and added.
__device__ __forceinline__ float wave_sum(float v) {
  v = dpp_add<0xB1>(v);
  v = dpp_add<0x4E>(v);
  v = dpp_add<0x141>(v);
  v = dpp_add<0x140>(v);
  int iv = __float_as_int(v);
  float s = __int_as_float(__builtin_amdgcn_readlane(iv, 0));
  s += __int_as_float(__builtin_amdgcn_readlane(iv, 16));
  s += __int_as_float(__builtin_amdgcn_readlane(iv, 32));
  s += __int_as_float(__builtin_amdgcn_readlane(iv, 48));
  return s;
}

// Number of set bits of a wave ballot below this lane (v_mbcnt_lo/hi).
__device__ __forceinline__ int ballot_rank(uint64_t ballot) {
  return (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(ballot >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)ballot, 0u));
}

// Inclusive prefix sum of one int per lane across the wave.
__device__ __forceinline__ int wave_scan_inclusive(int v, int lane) {
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    int o = __shfl_up(v, d, kWave);
    if (lane >= d) v += o;
  }
  return v;
}

}  // namespace cats
