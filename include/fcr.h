/*
 * fcr.h -- C ABI of libfcr.so, the MI355X (gfx950) column reduction of softmax attention.
 *
 * The reference has no FFI of its own: its hot path is a Python function that launches a
 * Triton kernel (flash_colreduce/flash.py:277-308, called from flash.py:375).  These entry
 * points are what a binding for that path has to call; each comment names the reference code
 * the entry point stands in for.
 *
 * Conventions
 *   - All pointers are DEVICE pointers on the current HIP device.  The library never
 *     allocates, frees or keeps them.
 *   - q is [B,H,M,D], k is [B,H,N,D], fp16, bf16 or fp32 elements (dtype below).  Strides are in
 *     ELEMENTS, order (batch, head, row, d); the d stride must be 1, row/head/batch strides must be
 *     multiples of 16 bytes (8 16-bit elements, 4 floats) and the base pointers 16-byte aligned; a row
 *     must be a multiple of 16 bytes and at most 1 KiB long: D a multiple of 8 in [8, 512] for
 *     16-bit elements, a multiple of 4 in [4, 256] for fp32.  Rows must not overlap (row stride >= D).
 *     (The reference takes any strides, flash.py:292-299; a caller with other layouts makes a
 *     contiguous, zero-padded copy first -- the Python host does.)  fp32 operands are multiplied at
 *     full precision and range (the reference's tl.dot rounds them to TF32, flash.py:59,108).
 *   - lse is fp32 [B*H, M] contiguous: per query row, log2(sum_j 2^(scale*log2(e)*<q_i,k_j>))
 *     over the keys the row may see.  It is the hand-over between the two kernels.  The buffer
 *     fcr_row_lse / fcr_colreduce write it to must be fcr_lse_bytes(B,H,M,N,D) long (scratch follows
 *     the result); fcr_col_reduce only reads the first B*H*M floats.
 *   - out is fp32 [B*H, N] contiguous and is fully overwritten (no zero-fill needed, unlike the
 *     atomically accumulated buffer at flash.py:286).
 *   - causal != 0 applies the right-aligned mask: key j takes part in row i iff
 *     j <= i + max(N-M, 0)   (flash.py:22-27, 198-207; naive.py:20-24).
 *   - stream is a hipStream_t (NULL = the default stream).  Launches are asynchronous.
 *   - Return value: 0 on success; negative FCR_E_* for a rejected argument (nothing was
 *     launched); positive = the hipError_t of a failed launch.  fcr_last_error() returns a
 *     thread-local, human readable description of the last non-zero return on this thread.
 *   - Thread safety: no mutable global state except the thread-local error text, the switches of
 *     fcr_set_option and the per-device record of the stream that ran the last single sweep (below); calls
 *     from several threads or streams do not interfere (each call needs its own lse / workspace buffer
 *     while it runs).
 */
#ifndef FCR_H
#define FCR_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FCR_VERSION 320 /* major*10000 + minor*100 + patch */

/* element type of q and k */
#define FCR_DTYPE_F16 0
#define FCR_DTYPE_BF16 1
#define FCR_DTYPE_F32 2 /* fp32 operands on the fp32 matrix instructions: D a multiple of 4, at most 256 */

/* column reduction over query rows */
#define FCR_REDUCE_SUM 0 /* also the numerator of 'mean' (flash.py:121-122) */
#define FCR_REDUCE_MAX 1 /* flash.py:123-124 */
#define FCR_REDUCE_MEAN 2 /* fcr_colreduce_to and fcr_colreduce_sum_max_to only: the sums divided as in flash.py:377-384 */

/* argument errors */
#define FCR_E_NULL -1      /* a required pointer is NULL */
#define FCR_E_DTYPE -2     /* dtype is not FCR_DTYPE_* */
#define FCR_E_SHAPE -3     /* B,H,M,N < 1, a row of D elements longer than 1 KiB or not a multiple of 16 bytes, sizes overflow */
#define FCR_E_STRIDE -4    /* d stride != 1 or a stride / base pointer breaks 16-byte alignment */
#define FCR_E_REDUCTION -5 /* reduction is not FCR_REDUCE_* */
#define FCR_E_SCALE -6     /* scale is not finite */
#define FCR_E_SCRATCH -7   /* fcr_colreduce_static: the problem needs more than FCR_STATIC_SCRATCH_BYTES */
#define FCR_E_WAIT -8      /* fcr_colreduce_status: a workgroup of the single sweep gave up waiting for its team */

/* fcr_set_option */
#define FCR_OPT_SINGLE_SWEEP 0 /* 0: few queries against many keys take the two kernels as well (default 1) */
#define FCR_OPT_WAIT_POLLS 1   /* polls of a team's slots after which a workgroup gives up (default 2^20) */

/* size of the built-in scratch buffer of fcr_colreduce_static, per GPU */
#define FCR_STATIC_SCRATCH_BYTES (16u << 20)

/* Library version (FCR_VERSION it was built from). */
int fcr_version(void);

/* Text for the last non-zero return value on the calling thread ("" if none). */
const char* fcr_last_error(void);

/*
 * Bytes the lse buffer of fcr_row_lse / fcr_colreduce must have for a problem, whatever its dtype and
 * D.  The first B*H*M floats are the result; scratch follows for few query rows against many keys: the
 * partial results of the row kernel when it splits the keys of a tile over several workgroups, or the
 * slots in which the workgroups of the single sweep publish their row sums (they depend on the number
 * of compute units: call this with the operands' device current).  0 for an empty problem.
 */
size_t fcr_lse_bytes(int B, int H, int M, int N, int D);

/*
 * First kernel: per-row base-2 log-sum-exp over all visible keys.
 * Stands in for the first half of the reference kernel: the two _update_softmax_lse sweeps and
 * "lse = m + log2(l)" (flash.py:35-80, 209-242), with scale*log2(e) folded as at flash.py:291.
 */
int fcr_row_lse(const void* q, const void* k, float* lse, int dtype, int B, int H, int M, int N,
                int D, const int64_t q_strides[4], const int64_t k_strides[4], float scale,
                int causal, void* stream);

/*
 * Second kernel: out[bh, j] = reduce_i 2^(scale*log2(e)*<q_i,k_j> - lse[bh, i]) over the rows
 * that may see key j; reduce = sum or max.  One workgroup owns a tile of key columns for the
 * whole sweep over query rows, so there are no atomics.
 * Stands in for the _update_softmax_cstats sweeps and their atomic_add / atomic_max
 * (flash.py:83-126, 244-274).
 */
int fcr_col_reduce(const void* q, const void* k, const float* lse, float* out, int dtype, int B,
                   int H, int M, int N, int D, const int64_t q_strides[4],
                   const int64_t k_strides[4], float scale, int reduction, int causal,
                   void* stream);

/*
 * Second kernel producing the column sums and the column maxima from ONE sweep (the reference needs two
 * full calls for that, flash.py:311-385 once per reduction).  out_sum and out_max are fp32 [B*H, N].
 */
int fcr_col_reduce_sum_max(const void* q, const void* k, const float* lse, float* out_sum, float* out_max,
                           int dtype, int B, int H, int M, int N, int D, const int64_t q_strides[4],
                           const int64_t k_strides[4], float scale, int causal, void* stream);

/*
 * Keep-mask of the k largest of every row of a contiguous fp32 [rows, N] (e.g. the [B*H, N] result of
 * the calls above): mask[r, j] = 1 for exactly min(max(k,0), N) columns of row r, 0 elsewhere; among
 * equal values the lower column wins.  threshold (optional, may be NULL) receives the k-th largest
 * value of each row.  No counterpart in the reference: it is the step its pruning callers take on
 * the reduced columns (README.md:9).  A NaN of either sign ranks above +inf (the order of torch.topk),
 * NaNs tie with each other; -0 and +0 are one value.  A threshold that is a NaN is stored as a NaN.
 */
int fcr_topk_mask(const float* scores, uint8_t* mask, float* threshold, int64_t rows, int N, int k, void* stream);

/*
 * fcr_topk_mask with scratch memory, for long rows: with ws_bytes >= fcr_topk_bytes(rows, N) > 0 a row of
 * more than 32768 columns is spread over workgroups of 8192 columns (five launches: four digits of a
 * radix select, then the mask) instead of being walked by one workgroup; same result, bit for bit.
 * fcr_topk_bytes returns 0 where the scratch would not be used (N <= 32768); with ws NULL or too small
 * the call is fcr_topk_mask.  ws must be 16-byte aligned; its contents before and after are irrelevant.
 */
size_t fcr_topk_bytes(int64_t rows, int N);
int fcr_topk_mask_ws(const float* scores, uint8_t* mask, float* threshold, int64_t rows, int N, int k, void* ws,
                     size_t ws_bytes, void* stream);

/*
 * The same for score rows of any FCR_DTYPE_* element type: fp16 and bf16 rows, as fcr_colreduce_to stores
 * them for 16-bit operands, are read as they are (order and ties of the stored values; threshold stays
 * fp32).  ws may be NULL (then ws_bytes is ignored); fcr_topk_bytes does not depend on the type.
 */
int fcr_topk_mask_typed(const void* scores, int dtype, uint8_t* mask, float* threshold, int64_t rows, int N, int k,
                        void* ws, size_t ws_bytes, void* stream);

/*
 * A faster and less exact alternative to FCR_DTYPE_F32 for fp32 operands whose values fit fp16 (the
 * 16-bit matrix instructions run at 16 times the fp32 rate): packs a contiguous fp32 [rows, D] into the fp16 [rows, terms * Dp] (Dp = D rounded up
 * to 8, zero padded) that the kernels above take with D' = terms * Dp and dtype FCR_DTYPE_F16.
 * terms = 3 writes [hi | hi | lo] for queries (is_key = 0) and [hi | lo | hi] for keys (is_key != 0),
 * hi = fp16(x), lo = fp16(x - hi): the kernels then see q.k to about 2^-22.  terms = 1 writes [hi].
 * terms * Dp must be <= 256; values beyond the fp16 range overflow.  scale must be passed explicitly
 * to the kernels (1/sqrt(D) of the original D).  The reference feeds fp32 straight to tl.dot
 * (flash.py:59,108), which on its hardware rounds both operands to TF32.
 */
int fcr_pack_f32(const float* src, void* dst, int64_t rows, int D, int terms, int is_key, void* stream);

/*
 * Both kernels back to back on one stream: the whole of _flash_colreduce (flash.py:277-308)
 * except the final cast to the input dtype, which stays with the host.  lse_ws is scratch of
 * fcr_lse_bytes(B,H,M,N,D) bytes whose first B*H*M floats hold the row statistics on return.
 */
int fcr_colreduce(const void* q, const void* k, float* out, float* lse_ws, int dtype, int B, int H,
                  int M, int N, int D, const int64_t q_strides[4], const int64_t k_strides[4],
                  float scale, int reduction, int causal, void* stream);

/*
 * fcr_colreduce for the column sums AND the column maxima of one problem (the reference makes two full calls,
 * flash.py:311-385 once per reduction): one row pass and one column sweep, or, for few queries against many
 * keys, one single sweep.  out_sum and out_max are fp32 [B*H, N]; lse_ws as for fcr_colreduce.
 */
int fcr_colreduce_sum_max(const void* q, const void* k, float* out_sum, float* out_max, float* lse_ws, int dtype, int B,
                          int H, int M, int N, int D, const int64_t q_strides[4], const int64_t k_strides[4],
                          float scale, int causal, void* stream);

/*
 * The whole operator as the reference's caller sees it: both kernels, the cast of the fp32 accumulation
 * to the result type (flash.py:308) and, for FCR_REDUCE_MEAN, the division of the sums (flash.py:377-384),
 * all inside the column kernel's store, so a call is two launches (three when the row sweep splits the
 * keys) whatever the reduction.  out is [B*H, N] of out_dtype (FCR_DTYPE_F16 / BF16 / F32; the reference
 * uses the operands' type).  The mean follows the reference's arithmetic step by step: the sum is rounded
 * to out_dtype first; columns left of the causal offset max(N-M,0) (every column without the mask) are
 * multiplied by the fp32 reciprocal of M; column j from the offset on is divided by N-j rounded to
 * out_dtype, the quotient rounded to out_dtype.  lse_ws as for fcr_colreduce.
 */
int fcr_colreduce_to(const void* q, const void* k, void* out, int out_dtype, float* lse_ws, int dtype, int B,
                     int H, int M, int N, int D, const int64_t q_strides[4], const int64_t k_strides[4],
                     float scale, int reduction, int causal, void* stream);

/*
 * fcr_colreduce without the lse_ws argument, for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference, whose launcher allocates with torch on every call (flash.py:286).  The row statistics and
 * the split row sweep's partial results live in a buffer of FCR_STATIC_SCRATCH_BYTES that is part of
 * the library's device image: every GPU the library runs on holds one until the process ends.  The call
 * allocates and frees nothing.  Problems with fcr_lse_bytes(B,H,M,N,D) > FCR_STATIC_SCRATCH_BYTES are
 * rejected with FCR_E_SCRATCH (16 MiB covers B*H*M <= 4 Mi rows when the keys are not split, e.g.
 * 32 heads of 131072 queries).  All calls on one GPU share the buffer: calls that overlap in time on one
 * GPU (different streams or threads) race; calls on one stream are ordered and safe.  The first call on
 * a device asks the runtime for the buffer's address and should be made outside graph capture.
 * Results are bitwise those of fcr_colreduce.
 */
/*
 * fcr_colreduce_sum_max with the tail of the reference's wrapper, as fcr_colreduce_to has it: both results
 * leave the kernel as [B*H, N] of out_dtype, and with sum_reduction = FCR_REDUCE_MEAN (else FCR_REDUCE_SUM)
 * the sums are divided as in flash.py:377-384.  Stands for two calls of flash_colreduce, 'sum' or 'mean' and
 * 'max' (flash.py:311-385), bit for bit what those give up to the order of the fp32 additions.
 */
int fcr_colreduce_sum_max_to(const void* q, const void* k, void* out_sum, void* out_max, int out_dtype, float* lse_ws,
                             int dtype, int B, int H, int M, int N, int D, const int64_t q_strides[4],
                             const int64_t k_strides[4], float scale, int sum_reduction, int causal, void* stream);

int fcr_colreduce_static(const void* q, const void* k, float* out, int dtype, int B, int H, int M, int N,
                         int D, const int64_t q_strides[4], const int64_t k_strides[4], float scale,
                         int reduction, int causal, void* stream);

/*
 * Few queries against many keys (M <= 128, N >= 1024, 16-bit elements, rows of at most 256 bytes): the calls
 * that run both kernels (fcr_colreduce, fcr_colreduce_to, fcr_colreduce_static) then take ONE sweep that
 * reads the keys once, where the reference's kernel reads them twice (flash.py:209-274).  Its workgroups
 * share a (b,h) pair and meet on counters in the workspace; a workgroup whose partners do not arrive
 * within FCR_OPT_WAIT_POLLS polls (only possible when the GPU cannot run the whole launch at once, e.g.
 * under a CU mask) stores NaN columns for that pair, sets a word in the workspace and goes on.
 * fcr_colreduce_status waits for the stream and returns FCR_E_WAIT if that happened in the last call that
 * used lse_ws with these sizes, 0 otherwise (also for problems that do not take the single sweep).
 * A single sweep fills the chip, one workgroup per CU, and two of them dispatched side by side would
 * starve each other until their waits run out.  Inside a process the library prevents that: a single
 * sweep issued on another stream than the previous one is made to wait on the GPU (an event recorded on
 * that stream, hipStreamWaitEvent on the new one; the host does not block, calls that stay on one stream
 * pay nothing).  Outside its reach: launches recorded under stream capture (graphs that hold single
 * sweeps must not replay side by side on one GPU), other processes on the same GPU, and
 * fcr_colreduce_static, whose calls must not overlap anyway.  There, switch the single sweep off or
 * keep such calls apart.
 * No counterpart in the reference, whose kernel has no cross-program dependencies.
 */
int fcr_colreduce_status(const float* lse_ws, int dtype, int B, int H, int M, int N, int D, void* stream);

/*
 * Process-wide switches (FCR_OPT_*), read by every later call: the single sweep on or off (results agree
 * to rounding either way) and the bound on its waits.  For tests and comparisons; returns 0 or FCR_E_SHAPE.
 */
int fcr_set_option(int option, long long value);

#ifdef __cplusplus
}
#endif
#endif /* FCR_H */
