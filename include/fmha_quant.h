/*
 * C ABI of the quantisation front end and back end of the INT8 attention path on MI355X (gfx950): what a caller does
 * to fp32 tensors before FMHAInferI8 and to its int8 output afterwards.  The reference does these steps on the host,
 * element by element (inc/utils.hpp:23-39,53; test_fmha_i8.cpp:91-110); here they are HBM-bound device kernels in the
 * same library (libfmha_i8.so), so that a pipeline never leaves the GPU between the float producer and the attention
 * kernel.  Same results, bit for bit, as the reference's host functions.
 *
 * All pointers are device pointers owned by the caller; x and out must be 16-byte aligned (hipMalloc gives 256), n is
 * any non-negative element count.  Every call enqueues kernels on `stream` and returns without synchronising; nothing
 * is allocated.  Return value: FMHA_I8_OK, FMHA_I8_ERR_NULL_POINTER, FMHA_I8_ERR_ALIGNMENT, FMHA_I8_ERR_SCALE (see
 * fmha_i8.h), or FMHA_I8_ERR_HIP_BASE + hipError_t.
 */
#ifndef FMHA_QUANT_H_
#define FMHA_QUANT_H_

#include <stdint.h>
#include <hip/hip_runtime_api.h>
#include "fmha_i8.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Replaces abs_max (inc/utils.hpp:31-39): *amax_out = max |x[i]| over n floats, 0 for n == 0; NaNs are skipped, as the
 * reference's `abs_val > max_val` skips them.  amax_out is one float in device memory: it can feed FMHAQuantizeI8 and,
 * copied to the host, FMHAParamI8. */
int FMHAAbsMaxF32(hipStream_t stream, const float* x, long long n, float* amax_out);

/* Replaces float_quant2_int8 applied over a tensor (inc/utils.hpp:23-29, test_fmha_i8.cpp:91-110):
 * out[i] = clamp(floorf(x[i] * (127 / amax) + 0.5), -127, 127), with the reference's float rounding at every step.
 * amax is read from device memory when amax_dev != NULL (no host round trip after FMHAAbsMaxF32), else amax_host is
 * used.  A NaN product (0 * inf when amax == 0) quantises to 0. */
int FMHAQuantizeI8(hipStream_t stream, const float* x, long long n, float amax_host, const float* amax_dev, int8_t* out);

/* The de-quantisation the reference prints and scores with (inc/utils.hpp:53,70): out[i] = (float)x[i] / 127 * amax. */
int FMHADequantizeI8(hipStream_t stream, const int8_t* x, long long n, float amax, float* out);

/* The same three steps for bfloat16 tensors (raw 16-bit patterns; torch.bfloat16 storage).  A bfloat16 widens to a
 * float exactly, so the results are those of the float functions above applied to the widened values; the de-quantised
 * value is rounded to bfloat16 once, to nearest even.  (The reference's driver only has float tensors,
 * test_fmha_i8.cpp:58-62; a bfloat16 producer would otherwise pay a widening pass over HBM first.) */
int FMHAAbsMaxBF16(hipStream_t stream, const uint16_t* x, long long n, float* amax_out);
int FMHAQuantizeI8BF16(hipStream_t stream, const uint16_t* x, long long n, float amax_host, const float* amax_dev,
                       int8_t* out);
int FMHADequantizeI8BF16(hipStream_t stream, const int8_t* x, long long n, float amax, uint16_t* out);

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* FMHA_QUANT_H_ */
