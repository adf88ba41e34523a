/*
 * C ABI of the gfx950 fused multi-head attention launchers.
 *
 * These entry points take the place of the two launchers the reference
 * declares in include/fused_mha.h:1-6 (defined at
 * kernel/fused_mha_kernel.cu:891-916).  Plain pointers and sizes only: no
 * torch types, so any host language can bind them (ctypes, cgo, JNI ...).
 *
 * Conventions shared by every entry point
 *   - q, k, v, o, d_o, d_q, d_k, d_v: dense fp16 tensors of shape
 *     (batch, n, head, d), element offset ((b*n + i)*head + h)*d + j
 *     (reference: kernel/fused_mha_kernel.cu:57-59).
 *   - lse: dense fp32 (batch, head, n): natural-log logsumexp of the scaled,
 *     masked score row, i.e. max + ln(sum) of the two statistics the
 *     reference stores separately (kernel/fused_mha_kernel.cu:298-303).
 *   - m == n (self attention, reference: kernel/fused_mha_api.cpp:68-69),
 *     d is 64 or 128.  Any n > 0 is accepted: the last, partial tile is
 *     handled inside the kernels, so callers need not right-pad the sequence
 *     to a multiple of 32 as the reference asks (README.md:3).
 *   - causal != 0: key j is visible to query i iff j <= i
 *     (reference: test.py:15-19).
 *   - stream is a hipStream_t passed as void*; NULL is the default stream.
 *     All work is enqueued asynchronously; nothing synchronises.
 *   - All pointers are borrowed device pointers and must be 16-byte aligned.
 *   - Size limits (FUSED_MHA_ERR_TOO_LARGE otherwise): n < 2^29, head * d < 2^24,
 *     ceil(n / 128) * batch * head < 2^23 and batch * head * n * d / 8 < 2^32.
 *   - Return value: FUSED_MHA_OK (0) or a negative FUSED_MHA_ERR_* code.
 *     Arguments are validated before anything is launched; only
 *     FUSED_MHA_ERR_LAUNCH can come back after part of the work (an earlier
 *     pass of the backward) has been enqueued.
 */
#ifndef FUSED_MHA_H_
#define FUSED_MHA_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FUSED_MHA_OK 0
#define FUSED_MHA_ERR_NULL_POINTER (-1)   /* a required pointer is NULL            */
#define FUSED_MHA_ERR_BAD_SHAPE (-2)      /* batch/head/n <= 0, m != n              */
#define FUSED_MHA_ERR_BAD_HEAD_DIM (-3)   /* d is neither 64 nor 128               */
#define FUSED_MHA_ERR_MISALIGNED (-4)     /* a pointer is not 16-byte aligned      */
#define FUSED_MHA_ERR_LAUNCH (-5)         /* the HIP runtime refused the launch    */
#define FUSED_MHA_ERR_BAD_SCALE (-6)      /* scale is NaN or infinite              */
#define FUSED_MHA_ERR_TOO_LARGE (-7)      /* beyond the limits listed below        */
#define FUSED_MHA_ERR_BAD_STRIDE (-8)     /* see fused_mha_strides                 */
#define FUSED_MHA_ERR_SCRATCH_LIMIT (-9)  /* see fused_mha_backward_noalloc        */
#define FUSED_MHA_ERR_RUNTIME (-10)       /* a HIP runtime query failed            */

/* Largest batch*head*n fused_mha_backward_noalloc accepts (8 MiB of scratch). */
#define FUSED_MHA_NOALLOC_MAX_ROWS (1 << 20)

/*
 * Element strides of a (batch, n, head, d) tensor whose last dimension is
 * contiguous: element (b, i, h, j) sits at b*batch + i*seq + h*head + j.
 * The dense layout is {n*head*d, head*d, d}.  Each stride must be a
 * non-negative multiple of 8 (rows start on 16-byte boundaries), seq below
 * 2^24 and head below 2^31.
 */
typedef struct fused_mha_strides {
  long long batch;
  long long seq;
  long long head;
} fused_mha_strides;

/*
 * Forward: o = softmax(scale * q k^T  [+ causal mask]) v, lse = row logsumexp.
 * Replaces fused_mha_forward (reference include/fused_mha.h:1-2); differs in
 * writing one logsumexp tensor instead of max_ptr and sum_ptr, in returning an
 * error code, and in accepting d = 64 as well as 128.
 */
int fused_mha_forward(const void *query_ptr, const void *key_ptr, const void *value_ptr,
                      void *output_ptr, void *lse_ptr,
                      int batch, int head, int m, int n, int d,
                      float scale, int causal, void *stream);

/*
 * The same for inputs that are not dense: q, k and v each come with their own
 * strides (NULL = dense), e.g. the three slices of a packed (batch, n, 3, head,
 * d) projection or (batch, head, n, d)-backed views; o and lse are written
 * dense.  No counterpart in the reference, whose Python side copies such inputs
 * (flash_attn_interface.py:14-15) and whose kernel assumes the dense layout
 * (kernel/fused_mha_kernel.cu:57-59); it is for callers that want to skip that
 * copy.
 */
int fused_mha_forward_strided(const void *query_ptr, const fused_mha_strides *query_strides,
                              const void *key_ptr, const fused_mha_strides *key_strides,
                              const void *value_ptr, const fused_mha_strides *value_strides,
                              void *output_ptr, void *lse_ptr,
                              int batch, int head, int n, int d,
                              float scale, int causal, void *stream);

/* Largest dS spill (bytes) the backward will use; beyond it the recompute path runs. */
#define FUSED_MHA_SPILL_MAX_BYTES ((size_t)16 << 30)

/*
 * Bytes of device scratch the backward works best with for this problem size.
 * The workspace starts with delta = rowsum(d_o * o) and lse * log2(e), both
 * fp32 of shape (batch, head, n), delta first: that much
 * (fused_mha_backward_min_workspace_bytes) is always needed.  When the
 * workspace also has room for the fp16 dS tiles (batch * head * np * np
 * elements, np = n rounded up to 128; at most FUSED_MHA_SPILL_MAX_BYTES), the
 * dK/dV pass writes the dS it forms there and the dQ pass is a single GEMM over
 * them: five GEMMs are executed, as in the reference's one-pass backward
 * (kernel/fused_mha_kernel.cu:564-713), instead of seven.  With the minimum
 * workspace the dQ pass recomputes S and dP.  Both paths are deterministic and
 * give the same dK and dV bits; dQ differs by summation order only.
 * fused_mha_backward_workspace_bytes returns the larger size when the spill is
 * within the limit, else the minimum; any size in between selects the
 * recompute path.  Both return 0 for an invalid shape.  No counterpart in the
 * reference, which receives delta from Python (flash_attn_interface.py:43-44).
 */
size_t fused_mha_backward_workspace_bytes(int batch, int head, int n, int d);
size_t fused_mha_backward_min_workspace_bytes(int batch, int head, int n, int d);

/*
 * Backward: d_q, d_k, d_v of the forward above, given d_o, the forward's
 * output o and lse.  Replaces fused_mha_backward (reference
 * include/fused_mha.h:4-6); differs in taking lse instead of max_ptr/sum_ptr,
 * in computing delta itself into `workspace` (fp32 accumulation) instead of
 * receiving a fp16 d_ptr, and in not requiring d_q to be zero-filled: every
 * element of d_q, d_k and d_v is overwritten.
 */
int fused_mha_backward(const void *query_ptr, const void *key_ptr, const void *value_ptr,
                       const void *output_ptr, const void *d_output_ptr, const void *lse_ptr,
                       void *workspace, size_t workspace_bytes,
                       void *d_query_ptr, void *d_key_ptr, void *d_value_ptr,
                       int batch, int head, int m, int n, int d,
                       float scale, int causal, void *stream);

/*
 * The same with strides for q, k, v and d_o (NULL = dense); o, lse, d_q, d_k
 * and d_v are dense.  No counterpart in the reference (see
 * fused_mha_forward_strided).
 */
int fused_mha_backward_strided(const void *query_ptr, const fused_mha_strides *query_strides,
                               const void *key_ptr, const fused_mha_strides *key_strides,
                               const void *value_ptr, const fused_mha_strides *value_strides,
                               const void *output_ptr,
                               const void *d_output_ptr, const fused_mha_strides *d_output_strides,
                               const void *lse_ptr, void *workspace, size_t workspace_bytes,
                               void *d_query_ptr, void *d_key_ptr, void *d_value_ptr,
                               int batch, int head, int n, int d,
                               float scale, int causal, void *stream);

/*
 * fused_mha_backward without a workspace argument and without any allocation:
 * delta and lse*log2(e) go to a static device array inside the library
 * (2 * FUSED_MHA_NOALLOC_MAX_ROWS floats = 8 MiB, held by every GPU the library
 * runs on until the process ends).  No counterpart in the reference; it is for
 * callers that cannot allocate device memory: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  It calls no hipMalloc,
 * hipFree or allocating library routine; the first call on a device looks up
 * the array's device address (which may make the runtime load the code
 * object: make that one call outside graph capture), every later call only
 * launches the kernels fused_mha_backward launches for a workspace of
 * fused_mha_backward_min_workspace_bytes, with bit-identical results.
 *   - batch*head*n above FUSED_MHA_NOALLOC_MAX_ROWS: FUSED_MHA_ERR_SCRATCH_LIMIT.
 *   - The device that owns the tensors must be the current device.
 *   - All calls on one GPU share that GPU's array: calls that overlap in time
 *     on one GPU (two streams, two threads) race; serialise them.
 */
int fused_mha_backward_noalloc(const void *query_ptr, const void *key_ptr, const void *value_ptr,
                               const void *output_ptr, const void *d_output_ptr, const void *lse_ptr,
                               void *d_query_ptr, void *d_key_ptr, void *d_value_ptr,
                               int batch, int head, int m, int n, int d,
                               float scale, int causal, void *stream);

/*
 * The three passes fused_mha_backward enqueues, one entry point each, so a
 * caller can time them separately or, with the minimum workspace, put the dQ
 * pass and the dK/dV pass (then independent of each other, both depend on the
 * delta pass) on different streams.  Same conventions and workspace as fused_mha_backward.  No
 * counterpart in the reference, whose backward is a single kernel
 * (kernel/fused_mha_kernel.cu:904-916).
 *   delta : workspace[b][h][i] = sum_j d_o[b][i][h][j] * o[b][i][h][j]  (fp32),
 *           followed by lse * log2(e) in the same shape
 *   dq    : d_q, streaming key/value tiles per block of 128 queries
 *   dkdv  : d_k and d_v, streaming query/d_o tiles per block of 128 keys
 * With a workspace of fused_mha_backward_workspace_bytes (room for the dS
 * tiles) the dkdv pass also writes dS and the dq pass reads it: dq must then
 * run after dkdv, on the same workspace.
 */
int fused_mha_backward_delta(const void *output_ptr, const void *d_output_ptr, const void *lse_ptr,
                             void *workspace, size_t workspace_bytes,
                             int batch, int head, int n, int d, void *stream);
int fused_mha_backward_dq(const void *query_ptr, const void *key_ptr, const void *value_ptr,
                          const void *d_output_ptr, const void *lse_ptr,
                          void *workspace, size_t workspace_bytes, void *d_query_ptr,
                          int batch, int head, int n, int d, float scale, int causal, void *stream);
int fused_mha_backward_dkdv(const void *query_ptr, const void *key_ptr, const void *value_ptr,
                            const void *d_output_ptr, const void *lse_ptr,
                            void *workspace, size_t workspace_bytes,
                            void *d_key_ptr, void *d_value_ptr,
                            int batch, int head, int n, int d, float scale, int causal, void *stream);

/* Static, human-readable text for a FUSED_MHA_* code. */
const char *fused_mha_error_string(int code);

#ifdef __cplusplus
}
#endif

#endif /* FUSED_MHA_H_ */
