/*
 * recis_hip.h - C ABI of librecis_hip.so: the gfx950 (MI355X) implementation of
 * RecIS's sparse-embedding hot path.
 *
 * Every entry point takes plain device pointers and sizes (no torch types) and
 * an opaque `stream` (a hipStream_t; NULL = the legacy default stream). Unless
 * stated otherwise a call only enqueues work on that stream and returns; it
 * never synchronises the device. All functions return RECIS_OK (0) or an error
 * code, with a human-readable message available from recis_hip_last_error().
 *
 * Each declaration names the reference function it stands in for
 * (paths relative to the alibaba/RecIS tree). The reference dispatches on
 * `tensor.device().is_cuda()` inside each op; these are the device branches.
 */
#ifndef RECIS_HIP_H_
#define RECIS_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RECIS_HIP_ABI_VERSION 1

/* status codes */
#define RECIS_OK 0
#define RECIS_ERR_ARG 1      /* bad argument (shape, dtype, alignment, NULL)  */
#define RECIS_ERR_HIP 2      /* a HIP runtime call failed                     */
#define RECIS_ERR_STATE 3    /* object used in a state that does not allow it */
#define RECIS_ERR_CAPACITY 4 /* a fixed capacity would be exceeded            */

/* element types of row storage / gradients */
#define RECIS_F32 0
#define RECIS_BF16 1
#define RECIS_F16 2

/* combiners (csrc/ops/embedding_segment_reduce.h:8 has SUM, MEAN, TILE; MAX is
 * an addition with no reference counterpart) */
#define RECIS_SUM 0
#define RECIS_MEAN 1
#define RECIS_TILE 2
#define RECIS_MAX 3

/* flags */
#define RECIS_FLAG_REV_UNIQUE 1 /* caller guarantees reverse_indices has no duplicates */

/* bits of the device-side soft-error word (recis_hip_poll_device_errors) */
#define RECIS_DEVERR_INDEX_RANGE 1  /* an index fell outside [0, rows)        */
#define RECIS_DEVERR_OFFSETS 2      /* offsets not monotone / outside [0, B]  */
#define RECIS_DEVERR_TABLE_FULL 4   /* id-map probe sequence found no slot    */

const char* recis_hip_last_error(void);
int recis_hip_abi_version(void);

/* Synchronises the current device, returns the soft-error bits raised by
 * kernels since the last poll in *bits and clears them. */
int recis_hip_poll_device_errors(int* bits);

/* ------------------------------------------------------------------------- *
 * Pooling: ragged gather + segment reduce
 * ------------------------------------------------------------------------- */

/*
 * Forward of the ragged-mode pooling.
 * Replaces: segment_reduce_forward, csrc/ops/embedding_segment_reduce_kernel.cu:199-273
 *           (kernel :23-75).
 *   unique_emb       [U, D]  rows, emb_dtype
 *   weight           [B] per-occurrence weight (weight_dtype) or NULL (= 1)
 *   reverse_indices  [B] occurrence -> row of unique_emb (int32 or int64);
 *                    NULL means the identity (rows are already materialised
 *                    per occurrence, U == B)
 *   offsets          [S + 1] segment boundaries into the B occurrences
 *   out              SUM/MEAN/MAX: [S, D];  TILE: [B, D]   (out_dtype)
 *   argmax_out       MAX only: [S, D] int32, occurrence index (absolute, into
 *                    the B occurrences) of the winning row, -1 for an empty
 *                    segment; may be NULL when no backward is needed
 * SUM:  out[s] = sum_i w_i * emb[rev_i];  MEAN: the same divided by the segment
 * length (weights are not normalised); TILE: out[i] = w_i * emb[rev_i];
 * MAX: element-wise maximum of emb[rev_i] over the segment (weights ignored,
 * first occurrence wins ties, empty segment -> 0).
 * The output is fully written by the call (no pre-zeroing needed).
 */
int recis_segment_reduce_forward(const void* unique_emb, int emb_dtype,
                                 const void* weight, int weight_dtype,
                                 const void* reverse_indices, int rev_is64,
                                 const void* offsets, int off_is64, void* out,
                                 int out_dtype, int32_t* argmax_out, int64_t B,
                                 int64_t U, int64_t S, int64_t D, int mode,
                                 void* stream);

/*
 * Backward of the ragged-mode pooling: scatters the pooled gradient back to the
 * unique rows.
 * Replaces: segment_reduce_backward, csrc/ops/embedding_segment_reduce_kernel.cu:276-350
 *           (kernel :79-120).
 *   grad_out     SUM/MEAN/MAX: [S, D]; TILE: [B, D]   (grad_dtype)
 *   argmax       MAX only: what the forward wrote
 *   grad_unique  [U, D] (out_dtype); fully written by the call
 * Without RECIS_FLAG_REV_UNIQUE duplicates in reverse_indices are accumulated
 * with fp32 atomics and out_dtype must be RECIS_F32. With the flag (or
 * reverse_indices == NULL) every row is written by plain stores.
 */
int recis_segment_reduce_backward(const void* grad_out, int grad_dtype,
                                  const void* weight, int weight_dtype,
                                  const void* reverse_indices, int rev_is64,
                                  const void* offsets, int off_is64,
                                  const int32_t* argmax, void* grad_unique,
                                  int out_dtype, int64_t B, int64_t U, int64_t S,
                                  int64_t D, int mode, int flags, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* RECIS_HIP_H_ */
