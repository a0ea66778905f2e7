/*
 * C ABI of the MI355X (gfx950) INT8 fused multi-head flash-attention launch path.
 *
 * The library (libfmha_i8.so) exports plain C symbols: pointers, PODs by value and a HIP stream handle.  No C++
 * types, no torch types.  A C++ caller that was written against the reference's `gpuImpl::FMHAInferI8`
 * (inc/fmha_i8.h:7-15) compiles unchanged against the forwarding wrapper at the bottom of this header; the only
 * difference is that the stream is a hipStream_t.
 *
 * Data contract (reference: src/fmha_i8.cu:157-173, inc/fmha_i8.cuh:45,88-89,112-114,325):
 *   q, k, v, o     int8, device memory, [batch_num, head_num, seq_len, head_dim] row-major contiguous,
 *                  base pointers 16-byte aligned (hipMalloc gives 256); o must not alias an input.
 *   padding_mask   int8, device memory, [batch_num, seq_len] over key positions; a NONZERO byte means the key is
 *                  masked OUT (inc/fmha_i8.cuh:189-192).  No alignment requirement.
 *   ownership      caller owns every buffer; the callee allocates nothing, frees nothing, keeps no pointer.
 *   asynchrony     one kernel is enqueued on `stream`; the call returns immediately and never synchronises.
 *   threading      no mutable global state: callable concurrently from any host thread.
 *
 * Supported shapes: head_dim in {64, 128}; seq_len from 1 to 65536; batch_num, head_num >= 1.
 * (The reference's ladder, src/fmha_i8.cu:39-154, covers head_dim in {64,128} and eleven fixed seq_len values: 64, 128,
 * 192, 256, 320, 384, 448, 512, 1024, 2048, 4096.  All of them are covered here, and so is every other length.
 * As in the reference, the softmax works on blocks of 128 keys when seq_len is a multiple of 128 and on blocks of 64 keys
 * when it is another multiple of 64 - the block size is part of the numerics, because P is quantised against the
 * BLOCK-LOCAL row maximum.  A length that is not a multiple of 64 gives what the caller would get by padding K, V and
 * the mask to the next multiple of 64 with masked keys (the float row sum of the last block adds its terms in another
 * order, nothing else differs); the library does it without the copies and never reads past the last key.)
 *
 * Numerics follow the reference kernel (inc/fmha_i8.cuh:71-72,181-253,298-332): int32 Q.K^T, 1/sqrt(d) and
 * q_amax*k_amax/127^2 dequantisation, softmax over blocks of 128 (or 64) keys with the BLOCK-LOCAL row maximum,
 * P requantised to int8 in [-128, 0] with scale -128, int32 P.V, online (m, l, O) merge, O requantised with
 * v_amax/(128*o_amax), round-half-even, clamp to [-127, 127].  Rows whose keys are all masked produce 0.
 */
#ifndef FMHA_I8_H_
#define FMHA_I8_H_

#include <hip/hip_runtime_api.h>
#include "fmha_param_i8.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes of FMHAInferI8Status.  Values >= 1000 are 1000 + the hipError_t of the failed launch. */
#define FMHA_I8_OK 0
#define FMHA_I8_ERR_NULL_POINTER 1   /* q, k, v, padding_mask or o is NULL */
#define FMHA_I8_ERR_HEAD_DIM 2       /* head_dim not in {64, 128} */
#define FMHA_I8_ERR_SEQ_LEN 3        /* a seq_len (queries or keys) <= 0 or > 65536 */
#define FMHA_I8_ERR_BATCH_HEAD 4     /* batch_num or head_num <= 0, or the grid would exceed HIP limits */
#define FMHA_I8_ERR_ALIGNMENT 5      /* q, k, v or o not 16-byte aligned */
#define FMHA_I8_ERR_SCALE 6          /* an amax is not finite, o_amax <= 0, q_amax * k_amax < 0, or a derived scale
                                        (q_amax * k_amax / 127^2 / sqrt(d), v_amax / (128 * o_amax)) overflows */
#define FMHA_I8_ERR_HIP_BASE 1000

/* Replaces gpuImpl::FMHAInferI8 (inc/fmha_i8.h:7-15, src/fmha_i8.cu:157-173).
 * Same argument list and meaning; returns nothing, like the reference.  On an unsupported shape the reference
 * silently launches nothing (src/fmha_i8.cu:39-154); this entry point also leaves `o` untouched, and additionally
 * writes one diagnostic line to stderr.  `use_tcu` is accepted for signature compatibility: the reference's
 * `false` path is an empty kernel (inc/fmha_i8.cuh:337-342); here both values run the MFMA kernel. */
void FMHAInferI8(hipStream_t stream, FMHAParamI8 fmha_param, AttnDataDescriptor attn_desc, const void* q,
                 const void* k, const void* v, const void* padding_mask, void* o, bool use_tcu);

/* Same operation, but reports what the reference cannot (its launch is unchecked, src/fmha_i8.cu:82-84):
 * FMHA_I8_OK, one of FMHA_I8_ERR_*, or FMHA_I8_ERR_HIP_BASE + hipError_t.  Never prints, never aborts.
 * The hipError_t is the return value of this call's own kernel launch: the calling thread's "last error" is neither
 * read nor cleared, so an earlier failure of some unrelated HIP call is not reported here and stays visible to the
 * caller's own hipGetLastError(). */
int FMHAInferI8Status(hipStream_t stream, FMHAParamI8 fmha_param, AttnDataDescriptor attn_desc, const void* q,
                      const void* k, const void* v, const void* padding_mask, void* o, bool use_tcu);

/* Argument check only (no HIP call at all): what FMHAInferI8Status would return before launching.
 * Stands in for the reference's if/else ladder over (head_dim, seq_len) (src/fmha_i8.cu:39-154). */
int FMHAInferI8CheckArgs(FMHAParamI8 fmha_param, AttnDataDescriptor attn_desc, const void* q, const void* k,
                         const void* v, const void* padding_mask, const void* o);

/* Shape of a call whose queries and keys differ in number: what the reference lists as planned ("S_src != S_dst",
 * README.md:13) and its kernel cannot express (one SEQ_LEN template parameter sizes Q, K, V and the mask alike,
 * inc/fmha_i8.cuh:45,88-89). */
typedef struct FMHACrossAttnDescriptor {
  int batch_num;
  int seq_len_q;   /* rows of q and o per head: any count from 1 to 65536 */
  int seq_len_kv;  /* rows of k and v per head, and mask bytes per batch entry: any count from 1 to 65536 */
  int head_num;
  int head_dim;
} FMHACrossAttnDescriptor;

/* Attention of seq_len_q queries over seq_len_kv keys.  q, o: int8 [batch_num, head_num, seq_len_q, head_dim];
 * k, v: int8 [batch_num, head_num, seq_len_kv, head_dim]; padding_mask: int8 [batch_num, seq_len_kv].  Everything
 * else (scales, numerics, ownership, asynchrony, status codes) as for FMHAInferI8Status; the softmax block is 128 keys
 * when seq_len_kv, rounded up to a multiple of 64, is a multiple of 128, else 64.  Query rows are independent of each other, so with
 * seq_len_q == seq_len_kv this IS FMHAInferI8Status (same kernel, same launch), and a call on the first n query rows
 * of a self-attention problem gives the first n rows of its output. */
int FMHAInferI8Cross(hipStream_t stream, FMHAParamI8 fmha_param, FMHACrossAttnDescriptor desc, const void* q,
                     const void* k, const void* v, const void* padding_mask, void* o);

/* FMHAInferI8Cross with P on all 255 steps of a byte: P = rne(255 p) in [0, 255] where the reference's kernel has
 * rne(-128 p) in [-128, 0] (inc/fmha_i8.cuh:241,249) - the "uint8 x int8" variant that the reference lists as planned
 * and has no code for (README.md:15,186).  Same arguments, layouts, scales, status codes and asynchrony; the output
 * differs from FMHAInferI8Cross's by at most a few LSBs and is closer to the unquantised attention (P carries one bit
 * more).  About a tenth slower: the matrix unit multiplies signed bytes only, so the kernel computes with P - 128 and
 * adds 128 times the column sums of every V tile. */
int FMHAInferI8CrossFullRangeP(hipStream_t stream, FMHAParamI8 fmha_param, FMHACrossAttnDescriptor desc, const void* q,
                               const void* k, const void* v, const void* padding_mask, void* o);

/* Argument check only, no HIP call: what FMHAInferI8Cross would return before launching. */
int FMHAInferI8CrossCheckArgs(FMHAParamI8 fmha_param, FMHACrossAttnDescriptor desc, const void* q, const void* k,
                              const void* v, const void* padding_mask, const void* o);

/* Human-readable text for a status code returned by the functions above (static storage). */
const char* FMHAInferI8StatusString(int status);

/* Library build identification: "fmha_i8 gfx950 <variant>" (static storage). */
const char* FMHAInferI8Version(void);

#ifdef __cplusplus
} /* extern "C" */

/* Source compatibility with call sites written for the reference (test_fmha_i8.cpp:204,207,219,222). */
namespace gpuImpl {
inline void FMHAInferI8(hipStream_t stream, FMHAParamI8 fmha_param, AttnDataDescriptor attn_desc, const void* q,
                        const void* k, const void* v, const void* padding_mask, void* o, const bool use_tcu) {
  ::FMHAInferI8(stream, fmha_param, attn_desc, q, k, v, padding_mask, o, use_tcu);
}
}  // namespace gpuImpl
#endif

#endif /* FMHA_I8_H_ */
