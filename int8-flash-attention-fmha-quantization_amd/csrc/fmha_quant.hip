// Quantisation front end / back end of the INT8 attention path for gfx950: abs-max, fp32 -> int8, int8 -> fp32.
// The reference does these on the host, one element at a time (inc/utils.hpp:23-39,53); here they are streaming
// kernels whose only cost is HBM traffic: 128-bit loads, one wavefront instruction covers 1 KiB of contiguous input,
// a few thousand wavefronts in flight, no LDS except for the block reduction of the maximum.
#include <hip/hip_runtime.h>
#include <tuple>
#include <stdint.h>

#include "../../include/fmha_quant.h"

// Every float operation below must round exactly where the reference's host code rounds: no fused multiply-add.
#pragma clang fp contract(off)

namespace fmha_i8_gfx950 {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kQuantThreads = 256;
constexpr int kQuantUnroll = 4;          // 16-byte units per thread and loop trip: 64 B per lane in flight per trip
constexpr int kQuantMaxBlocks = 256 * 2; // two workgroups of 4 wavefronts per CU: measured best from 32 MiB to 1 GiB (more
                                         // workgroups lose up to 15 %, and every workgroup of the abs-max ends in an atomic)
constexpr long long kCacheBytes = 256ll << 20;  // beyond the last-level cache, streams bypass it (non-temporal): +18 %
                                                // at 1 GiB, -8 % at 128 MiB, hence the switch

__global__ void zero_float_kernel(float* p) { *p = 0.f; }

// inc/utils.hpp:31-39.  |x| of non-NaN floats orders like its bit pattern, so the grid-wide maximum is an unsigned
// atomic max on *out, which zero_float_kernel has cleared.
__global__ __launch_bounds__(kQuantThreads) void abs_max_kernel(const float* __restrict__ x, long long n,
                                                                 float* __restrict__ out) {
  const long long units = n / 4;
  const float4* __restrict__ x4 = reinterpret_cast<const float4*>(x);
  const long long stride = (long long)gridDim.x * kQuantThreads;
  float m = 0.f;
  auto take = [&](float v) {
    const float a = fabsf(v);
    m = a > m ? a : m;  // a NaN never compares greater: skipped, as in the reference
  };
  // (one running maximum: 16 compare-selects per 64 bytes are far below what the loads cost)
  long long j = (long long)blockIdx.x * kQuantThreads + threadIdx.x;
  for (; j + (kQuantUnroll - 1) * stride < units; j += kQuantUnroll * stride) {
    float4 v[kQuantUnroll];
#pragma unroll
    for (int u = 0; u < kQuantUnroll; ++u) v[u] = x4[j + u * stride];
#pragma unroll
    for (int u = 0; u < kQuantUnroll; ++u) { take(v[u].x); take(v[u].y); take(v[u].z); take(v[u].w); }
  }
  for (; j < units; j += stride) {
    const float4 v = x4[j];
    take(v.x); take(v.y); take(v.z); take(v.w);
  }
  if (blockIdx.x == 0 && threadIdx.x < (int)(n - 4 * units)) take(x[4 * units + threadIdx.x]);
  // wavefront, then workgroup, then grid
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float o = __shfl_xor(m, off);
    m = o > m ? o : m;
  }
  __shared__ float part[kQuantThreads / 64];
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 1; w < kQuantThreads / 64; ++w) m = part[w] > m ? part[w] : m;
    if (m > 0.f) atomicMax(reinterpret_cast<unsigned int*>(out), __float_as_uint(m));
  }
}

// inc/utils.hpp:23-29: floorf(x * (127 / amax) + 0.5) in float arithmetic (the reference's double add is exact and
// floorf takes a float, which is one correctly rounded float add), clamp to [-127, 127]; NaN -> 0.
__device__ __forceinline__ int quant1(float x, float scale) {
  const float q = floorf(x * scale + 0.5f);
  return (int)fminf(fmaxf(q, -127.f), 127.f);  // clamped as a float, so that an infinite product is +-127 too
}
__device__ __forceinline__ int quant1_nan0(float x, float scale) {
  const float p = x * scale;
  return p == p ? quant1(x, scale) : 0;
}

template <bool NT>
__global__ __launch_bounds__(kQuantThreads) void quantize_i8_kernel(const float* __restrict__ x, long long n,
                                                                     float amax_host,
                                                                     const float* __restrict__ amax_dev,
                                                                     int8_t* __restrict__ out) {
  const float amax = amax_dev != nullptr ? *amax_dev : amax_host;
  const float scale = 127.0f / amax;
  const long long units = n / 4;
  const v4f* __restrict__ x4 = reinterpret_cast<const v4f*>(x);
  int* __restrict__ o4 = reinterpret_cast<int*>(out);
  const long long stride = (long long)gridDim.x * kQuantThreads;
  auto pack = [&](const v4f& v) {
    return (quant1_nan0(v.x, scale) & 0xff) | ((quant1_nan0(v.y, scale) & 0xff) << 8) |
           ((quant1_nan0(v.z, scale) & 0xff) << 16) | (quant1_nan0(v.w, scale) << 24);
  };
  long long j = (long long)blockIdx.x * kQuantThreads + threadIdx.x;
  for (; j + (kQuantUnroll - 1) * stride < units; j += kQuantUnroll * stride) {
    v4f v[kQuantUnroll];
#pragma unroll
    for (int u = 0; u < kQuantUnroll; ++u) v[u] = NT ? __builtin_nontemporal_load(&x4[j + u * stride]) : x4[j + u * stride];
#pragma unroll
    for (int u = 0; u < kQuantUnroll; ++u) {
      if (NT) __builtin_nontemporal_store(pack(v[u]), &o4[j + u * stride]);
      else o4[j + u * stride] = pack(v[u]);
    }
  }
  for (; j < units; j += stride) o4[j] = pack(x4[j]);
  if (blockIdx.x == 0 && threadIdx.x < (int)(n - 4 * units))
    out[4 * units + threadIdx.x] = (int8_t)quant1_nan0(x[4 * units + threadIdx.x], scale);
}

// inc/utils.hpp:53: (float)v / 127.0f * amax, in that order.  The quotient is formed without the division sequence:
// q0 = v * fl(1/127), the exact remainder r = v - 127 q0 (one fma), q = q0 + r * fl(1/127) (one fma).  For each of the
// 256 values of v this is the correctly rounded v / 127.0f (checked exhaustively by the tests); a quarter of the
// instructions, and these kernels have to keep up with HBM.
__device__ __forceinline__ float dequant1(int v, float amax) {
  constexpr float kRcp127 = 1.0f / 127.0f;
  const float fv = (float)v;
  const float q0 = fv * kRcp127;
  const float r = __builtin_fmaf(-q0, 127.0f, fv);
  return __builtin_fmaf(r, kRcp127, q0) * amax;
}
template <bool NT>
__global__ __launch_bounds__(kQuantThreads) void dequantize_i8_kernel(const int8_t* __restrict__ x, long long n,
                                                                       float amax, float* __restrict__ out) {
  const long long units = n / 4;
  const int* __restrict__ x4 = reinterpret_cast<const int*>(x);
  v4f* __restrict__ o4 = reinterpret_cast<v4f*>(out);
  const long long stride = (long long)gridDim.x * kQuantThreads;
  auto one = [&](int v) { return dequant1(v, amax); };
  auto unpack = [&](int w) {
    return v4f{one((int8_t)(w & 0xff)), one((int8_t)((w >> 8) & 0xff)), one((int8_t)((w >> 16) & 0xff)), one(w >> 24)};
  };
  long long j = (long long)blockIdx.x * kQuantThreads + threadIdx.x;
  for (; j + (kQuantUnroll - 1) * stride < units; j += kQuantUnroll * stride) {
    int w[kQuantUnroll];
#pragma unroll
    for (int u = 0; u < kQuantUnroll; ++u) w[u] = NT ? __builtin_nontemporal_load(&x4[j + u * stride]) : x4[j + u * stride];
#pragma unroll
    for (int u = 0; u < kQuantUnroll; ++u) {
      if (NT) __builtin_nontemporal_store(unpack(w[u]), &o4[j + u * stride]);
      else o4[j + u * stride] = unpack(w[u]);
    }
  }
  for (; j < units; j += stride) o4[j] = unpack(x4[j]);
  if (blockIdx.x == 0 && threadIdx.x < (int)(n - 4 * units)) out[4 * units + threadIdx.x] = one(x[4 * units + threadIdx.x]);
}

// ---- bfloat16 tensors ---------------------------------------------------------------------------------------------
// A bfloat16 is the upper half of a float: widening is exact, so the three functions below are the float ones applied
// to the widened values (same roundings, same results); the de-quantised float is rounded to bfloat16 once, to nearest
// even.  One 16-byte unit holds eight elements.
typedef unsigned short v8h __attribute__((ext_vector_type(8)));
typedef unsigned short v4h __attribute__((ext_vector_type(4)));
typedef int v2i32 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float widen(unsigned short h) { return __uint_as_float((unsigned)h << 16); }
__device__ __forceinline__ unsigned short narrow_rne(float f) {
  const unsigned u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40u);  // NaN stays NaN
  return (unsigned short)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

__global__ __launch_bounds__(kQuantThreads) void abs_max_bf16_kernel(const unsigned short* __restrict__ x, long long n,
                                                                      float* __restrict__ out) {
  const long long units = n / 8;
  const v8h* __restrict__ x8 = reinterpret_cast<const v8h*>(x);
  const long long stride = (long long)gridDim.x * kQuantThreads;
  float m = 0.f;
  auto take = [&](unsigned short h) {
    const float a = fabsf(widen(h));
    m = a > m ? a : m;  // a NaN never compares greater: skipped
  };
  long long j = (long long)blockIdx.x * kQuantThreads + threadIdx.x;
  for (; j + (kQuantUnroll - 1) * stride < units; j += kQuantUnroll * stride) {
    v8h v[kQuantUnroll];
#pragma unroll
    for (int u = 0; u < kQuantUnroll; ++u) v[u] = x8[j + u * stride];
#pragma unroll
    for (int u = 0; u < kQuantUnroll; ++u)
#pragma unroll
      for (int e = 0; e < 8; ++e) take(v[u][e]);
  }
  for (; j < units; j += stride) {
    const v8h v = x8[j];
#pragma unroll
    for (int e = 0; e < 8; ++e) take(v[e]);
  }
  if (blockIdx.x == 0 && threadIdx.x < (int)(n - 8 * units)) take(x[8 * units + threadIdx.x]);
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float o = __shfl_xor(m, off);
    m = o > m ? o : m;
  }
  __shared__ float part[kQuantThreads / 64];
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 1; w < kQuantThreads / 64; ++w) m = part[w] > m ? part[w] : m;
    if (m > 0.f) atomicMax(reinterpret_cast<unsigned int*>(out), __float_as_uint(m));
  }
}

template <bool NT>
__global__ __launch_bounds__(kQuantThreads) void quantize_i8_bf16_kernel(const unsigned short* __restrict__ x, long long n,
                                                                          float amax_host,
                                                                          const float* __restrict__ amax_dev,
                                                                          int8_t* __restrict__ out) {
  const float amax = amax_dev != nullptr ? *amax_dev : amax_host;
  const float scale = 127.0f / amax;
  const long long units = n / 8;
  const v8h* __restrict__ x8 = reinterpret_cast<const v8h*>(x);
  v2i32* __restrict__ o8 = reinterpret_cast<v2i32*>(out);
  const long long stride = (long long)gridDim.x * kQuantThreads;
  auto q = [&](unsigned short h) { return quant1_nan0(widen(h), scale) & 0xff; };
  auto pack = [&](const v8h& v) {
    return v2i32{q(v[0]) | (q(v[1]) << 8) | (q(v[2]) << 16) | (q(v[3]) << 24),
                 q(v[4]) | (q(v[5]) << 8) | (q(v[6]) << 16) | (q(v[7]) << 24)};
  };
  long long j = (long long)blockIdx.x * kQuantThreads + threadIdx.x;
  for (; j + (kQuantUnroll - 1) * stride < units; j += kQuantUnroll * stride) {
    v8h v[kQuantUnroll];
#pragma unroll
    for (int u = 0; u < kQuantUnroll; ++u) v[u] = NT ? __builtin_nontemporal_load(&x8[j + u * stride]) : x8[j + u * stride];
#pragma unroll
    for (int u = 0; u < kQuantUnroll; ++u) {
      if (NT) __builtin_nontemporal_store(pack(v[u]), &o8[j + u * stride]);
      else o8[j + u * stride] = pack(v[u]);
    }
  }
  for (; j < units; j += stride) o8[j] = pack(x8[j]);
  if (blockIdx.x == 0 && threadIdx.x < (int)(n - 8 * units))
    out[8 * units + threadIdx.x] = (int8_t)quant1_nan0(widen(x[8 * units + threadIdx.x]), scale);
}

template <bool NT>
__global__ __launch_bounds__(kQuantThreads) void dequantize_i8_bf16_kernel(const int8_t* __restrict__ x, long long n,
                                                                            float amax, unsigned short* __restrict__ out) {
  const long long units = n / 8;
  const v2i32* __restrict__ x8 = reinterpret_cast<const v2i32*>(x);
  v8h* __restrict__ o8 = reinterpret_cast<v8h*>(out);
  const long long stride = (long long)gridDim.x * kQuantThreads;
  auto one = [&](int v) { return narrow_rne(dequant1(v, amax)); };
  auto unpack = [&](const v2i32& w) {
    v8h r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = one((int8_t)((w[e >> 2] >> (8 * (e & 3))) & 0xff));
    return r;
  };
  long long j = (long long)blockIdx.x * kQuantThreads + threadIdx.x;
  for (; j + (kQuantUnroll - 1) * stride < units; j += kQuantUnroll * stride) {
    v2i32 w[kQuantUnroll];
#pragma unroll
    for (int u = 0; u < kQuantUnroll; ++u) w[u] = NT ? __builtin_nontemporal_load(&x8[j + u * stride]) : x8[j + u * stride];
#pragma unroll
    for (int u = 0; u < kQuantUnroll; ++u) {
      if (NT) __builtin_nontemporal_store(unpack(w[u]), &o8[j + u * stride]);
      else o8[j + u * stride] = unpack(w[u]);
    }
  }
  for (; j < units; j += stride) o8[j] = unpack(x8[j]);
  if (blockIdx.x == 0 && threadIdx.x < (int)(n - 8 * units)) out[8 * units + threadIdx.x] = one(x[8 * units + threadIdx.x]);
}

inline int quant_blocks(long long n) {
  const long long want = (n / 4 + (long long)kQuantThreads * kQuantUnroll - 1) / ((long long)kQuantThreads * kQuantUnroll);
  return (int)(want < 1 ? 1 : (want > kQuantMaxBlocks ? kQuantMaxBlocks : want));
}
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
// Launches report the status of the launch itself (what hipLaunchKernel returns), not the calling thread's last
// error: an earlier failure that has nothing to do with this library is neither reported as ours nor cleared.
template <typename... Params, typename... Args>
inline hipError_t launch_kernel(void (*kernel)(Params...), int blocks, int threads, hipStream_t stream, Args... args) {
  std::tuple<Params...> by_value{static_cast<Params>(args)...};
  void* ptrs[sizeof...(Params)];
  int i = 0;
  std::apply([&](auto&... a) { ((ptrs[i++] = static_cast<void*>(&a)), ...); }, by_value);
  return hipLaunchKernel(reinterpret_cast<const void*>(kernel), dim3(blocks), dim3(threads), ptrs, 0, stream);
}
inline int status_of(hipError_t err) { return err == hipSuccess ? FMHA_I8_OK : FMHA_I8_ERR_HIP_BASE + (int)err; }

}  // namespace fmha_i8_gfx950

extern "C" {

int FMHAAbsMaxF32(hipStream_t stream, const float* x, long long n, float* amax_out) {
  using namespace fmha_i8_gfx950;
  if (amax_out == nullptr || (x == nullptr && n > 0) || n < 0) return FMHA_I8_ERR_NULL_POINTER;
  if (!aligned16(x)) return FMHA_I8_ERR_ALIGNMENT;
  hipError_t err = launch_kernel(zero_float_kernel, 1, 1, stream, amax_out);
  if (err == hipSuccess && n > 0) err = launch_kernel(abs_max_kernel, quant_blocks(n), kQuantThreads, stream, x, n, amax_out);
  return status_of(err);
}

int FMHAQuantizeI8(hipStream_t stream, const float* x, long long n, float amax_host, const float* amax_dev, int8_t* out) {
  using namespace fmha_i8_gfx950;
  if (n < 0 || ((x == nullptr || out == nullptr) && n > 0)) return FMHA_I8_ERR_NULL_POINTER;
  if (!aligned16(x) || !aligned16(out)) return FMHA_I8_ERR_ALIGNMENT;
  if (amax_dev == nullptr && !(amax_host == amax_host)) return FMHA_I8_ERR_SCALE;
  if (n == 0) return FMHA_I8_OK;
  if (5 * n > kCacheBytes)
    return status_of(launch_kernel(quantize_i8_kernel<true>, quant_blocks(n), kQuantThreads, stream, x, n, amax_host, amax_dev, out));
  return status_of(launch_kernel(quantize_i8_kernel<false>, quant_blocks(n), kQuantThreads, stream, x, n, amax_host, amax_dev, out));
}

int FMHADequantizeI8(hipStream_t stream, const int8_t* x, long long n, float amax, float* out) {
  using namespace fmha_i8_gfx950;
  if (n < 0 || ((x == nullptr || out == nullptr) && n > 0)) return FMHA_I8_ERR_NULL_POINTER;
  if (!aligned16(x) || !aligned16(out)) return FMHA_I8_ERR_ALIGNMENT;
  if (n == 0) return FMHA_I8_OK;
  if (5 * n > kCacheBytes)
    return status_of(launch_kernel(dequantize_i8_kernel<true>, quant_blocks(n), kQuantThreads, stream, x, n, amax, out));
  return status_of(launch_kernel(dequantize_i8_kernel<false>, quant_blocks(n), kQuantThreads, stream, x, n, amax, out));
}

int FMHAAbsMaxBF16(hipStream_t stream, const uint16_t* x, long long n, float* amax_out) {
  using namespace fmha_i8_gfx950;
  if (amax_out == nullptr || (x == nullptr && n > 0) || n < 0) return FMHA_I8_ERR_NULL_POINTER;
  if (!aligned16(x)) return FMHA_I8_ERR_ALIGNMENT;
  hipError_t err = launch_kernel(zero_float_kernel, 1, 1, stream, amax_out);
  if (err == hipSuccess && n > 0)
    err = launch_kernel(abs_max_bf16_kernel, quant_blocks(n / 2), kQuantThreads, stream, x, n, amax_out);
  return status_of(err);
}

int FMHAQuantizeI8BF16(hipStream_t stream, const uint16_t* x, long long n, float amax_host, const float* amax_dev,
                       int8_t* out) {
  using namespace fmha_i8_gfx950;
  if (n < 0 || ((x == nullptr || out == nullptr) && n > 0)) return FMHA_I8_ERR_NULL_POINTER;
  if (!aligned16(x) || !aligned16(out)) return FMHA_I8_ERR_ALIGNMENT;
  if (amax_dev == nullptr && !(amax_host == amax_host)) return FMHA_I8_ERR_SCALE;
  if (n == 0) return FMHA_I8_OK;
  if (3 * n > kCacheBytes)
    return status_of(launch_kernel(quantize_i8_bf16_kernel<true>, quant_blocks(n / 2), kQuantThreads, stream, x, n, amax_host, amax_dev, out));
  return status_of(launch_kernel(quantize_i8_bf16_kernel<false>, quant_blocks(n / 2), kQuantThreads, stream, x, n, amax_host, amax_dev, out));
}

int FMHADequantizeI8BF16(hipStream_t stream, const int8_t* x, long long n, float amax, uint16_t* out) {
  using namespace fmha_i8_gfx950;
  if (n < 0 || ((x == nullptr || out == nullptr) && n > 0)) return FMHA_I8_ERR_NULL_POINTER;
  if (!aligned16(x) || !aligned16(out)) return FMHA_I8_ERR_ALIGNMENT;
  if (n == 0) return FMHA_I8_OK;
  if (3 * n > kCacheBytes)
    return status_of(launch_kernel(dequantize_i8_bf16_kernel<true>, quant_blocks(n / 2), kQuantThreads, stream, x, n, amax, out));
  return status_of(launch_kernel(dequantize_i8_bf16_kernel<false>, quant_blocks(n / 2), kQuantThreads, stream, x, n, amax, out));
}

}  // extern "C"
