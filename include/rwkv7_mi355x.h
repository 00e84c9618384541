/* C ABI of librwkv7_mi355x.so: the RWKV7 generalized delta rule on MI355X (gfx950).
 *
 * Plain pointers and sizes only; every pointer is DEVICE memory owned by the caller
 * unless a comment says otherwise.  The library never allocates and never
 * synchronises; every call enqueues its kernels on the hipStream_t passed as `stream`
 * (NULL = the default stream) on the caller's current device and returns.  The only
 * state it keeps between calls is a process-wide launch counter (an atomic), from
 * which every chunked forward launch draws a fresh 64-bit tag; calls from several
 * threads are safe.
 *
 * Return value of every int function: 0 = ok, < 0 = argument error (RWKV7_ERR_*,
 * nothing was launched), > 0 = a hipError_t reported by a launch.
 *
 * Operator (per batch b and head h, state h[K][V] float32; K = V = 64 everywhere, K = V = 128 where a
 * function's comment says so):
 *     d_t  = exp(-exp(w_t))                      the API's `w` is NOT the log decay
 *     sa_t = a_t^T h_{t-1}
 *     h_t  = diag(d_t) h_{t-1} + b_t sa_t^T + k_t v_t^T
 *     o_t  = r_t^T h_t
 * as the reference's native loop defines it
 * (/root/reference/rwkv_ops/rwkv7_kernel/native_keras_op.py:58,85,87), with the
 * state in the kernel path's [N, H, K, V] layout
 * (/root/reference/README.md:66,
 *  /root/reference/rwkv_ops/rwkv7_kernel/triton_kernel/chunk_h_fwd.py:66-71).
 *
 * Tensor layout: r, w, k, v, a, b, o and their gradients are [B, T, H, 64]
 * contiguous in `dtype` (head_first callers permute in the host language, as
 * /root/reference/rwkv_ops/rwkv7_kernel/torch_op.py:451-455 does).  States and
 * state gradients are float32 [B, H, 64, 64] contiguous.  `h0` may be NULL (zero
 * state); `h0_batch_stride` is the element stride between batches of h0: H*64*64
 * normally, 0 to broadcast one [1, H, 64, 64] state over the batch
 * (native_keras_op.py:62-63).
 */
#ifndef RWKV7_MI355X_H
#define RWKV7_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 2: the one-kernel forward's workspace holds a status record, two state slots per (batch, head) and their
 * carriers (sizes from the *_workspace_bytes functions as before); rwkv7_set_giveup_notice; RWKV6 float32 gradients
 * 3: the RWKV6 entry points take K = V = 128; rwkv6_bwd_workspace_bytes_head */
#define RWKV7_ABI_VERSION 3

/* element type of r, w, k, v, a, b, o and the input gradients */
#define RWKV7_DTYPE_BF16 0
#define RWKV7_DTYPE_F32  1
#define RWKV7_DTYPE_F16  2   /* float16: read by the decode step and the float32 recurrent forward and backward
                              * only (values are widened on load, o and the gradients are rounded on store).
                              * rwkv7_fwd, rwkv7_fwd_gather and rwkv7_fwd_varlen therefore run the recurrent kernel
                              * for every T with it; the chunked kernels, rwkv7_bwd and the RWKV6 entry points
                              * answer RWKV7_ERR_UNSUPPORTED.  (The reference's kernel path casts float16 inputs to
                              * bfloat16, torch_op.py:451-455; callers who want that speed for long T do the
                              * same and pass RWKV7_DTYPE_BF16.) */

/* argument errors */
#define RWKV7_OK                 0
#define RWKV7_ERR_NULL_POINTER  -1   /* a required pointer is NULL */
#define RWKV7_ERR_BAD_DTYPE     -2   /* dtype is not RWKV7_DTYPE_* */
#define RWKV7_ERR_BAD_HEAD_SIZE -3   /* K != V, or a head size this entry point has no kernel for */
#define RWKV7_ERR_BAD_SHAPE     -4   /* B, T or H < 1, or a size overflows the kernels' index range */
#define RWKV7_ERR_BAD_STRIDE    -5   /* h0_batch_stride is neither 0 nor H*K*V */
#define RWKV7_ERR_WORKSPACE     -6   /* workspace NULL, misaligned (256 B) or smaller than *_workspace_bytes */
#define RWKV7_ERR_ALIGNMENT     -7   /* a tensor pointer is not 16-byte aligned */
#define RWKV7_ERR_UNSUPPORTED   -8   /* combination not built (see the function's comment) */
#define RWKV7_ERR_TOO_LARGE     -9   /* rwkv7_fwd_noalloc: B*H > RWKV7_NOALLOC_MAX_BH */

int rwkv7_abi_version(void);

/* Human-readable text for a status returned by this library (static storage). */
const char* rwkv7_status_string(int status);

/* ---- forward over a sequence ------------------------------------------------
 * Replaces the body of `generalized_delta_rule`
 * (/root/reference/rwkv_ops/rwkv7_kernel/torch_op.py:458-490): the cast, the
 * `-exp(w)` of chunk_rwkv7 (:433-434) and the six launches of chunk_dplr_fwd
 * (:46-120).  Writes o [B,T,H,64] (`dtype`) and, if ht != NULL, the final state.
 * bf16 runs the fused chunked MFMA kernel (one workgroup per 64-token chunk; the
 * state travels from chunk to chunk through the workspace) and needs a workspace of
 * rwkv7_fwd_workspace_bytes() (a few MB: two state slots of 17 KiB per
 * (batch, head)); f32 runs the chunked float32 kernel (16-token chunks on the float32
 * matrix cores, one workgroup per (batch, head) with the state in registers; float32
 * arithmetic throughout, the accuracy of the reference's native loop) and needs none (ws
 * may be NULL).  T == 1 takes the decode kernel for both types, and 2 <= T <= 12 the
 * recurrent kernel (a handful of tokens is faster one at a time with the state in registers
 * than through a chunk; float32 arithmetic, no workspace used).  Two calls that overlap
 * in time must not share a workspace.
 * K = V = 128 (the head size of /root/reference/test_script/test_rwkv7_value.py:51): accepted by
 * rwkv7_fwd, rwkv7_fwd_gather, rwkv7_fwd_varlen, rwkv7_fwd_noalloc, rwkv7_fwd_recurrent, the two decode-step
 * calls and rwkv7_bwd_recurrent.  bf16 with T > 12 runs a chunked MFMA kernel of its own (one workgroup per
 * (batch, head) walking the chunks with the state in registers; no workspace, ws may be NULL); float32, float16
 * and T <= 12 run the float32 recurrent kernel at this head size (0.5 to 1 us per token).  rwkv7_bwd and
 * rwkv7_bwd_varlen hand a call at this head size to rwkv7_bwd_recurrent / rwkv7_bwd_recurrent_varlen (any of the
 * three dtypes), whose workspace sizes apply: rwkv7_bwd_recurrent_workspace_bytes(B, T, H, 128) and
 * rwkv7_bwd_recurrent_varlen_workspace_bytes(n_seq, T_total, H, 128). */
size_t rwkv7_fwd_workspace_bytes(int B, int T, int H, int dtype);
int rwkv7_fwd(const void* r, const void* w, const void* k, const void* v,
              const void* a, const void* b,
              const float* h0, int64_t h0_batch_stride,
              void* o, float* ht,
              int B, int T, int H, int K, int V, int dtype,
              void* ws, size_t ws_bytes, void* stream);

/* ---- the forward without a workspace argument ---------------------------------------
 * No counterpart in the reference.  For callers that cannot allocate device memory
 * around the call -- code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc -- and so cannot provide rwkv7_fwd's workspace: the same forward,
 * same arguments and results, with the workspace taken from a static device array
 * inside the library (8.5 MiB, held on every GPU the library is loaded on until the
 * process ends).  That array holds the one-kernel form's hand-off slots and status record
 * for up to RWKV7_NOALLOC_MAX_BH (batch, head) sequences, so B*H beyond that is refused
 * with RWKV7_ERR_TOO_LARGE; T is not limited.  bf16 with T > 12 always takes the
 * one-kernel chunked form here (rwkv7_fwd prefers two kernels below 72 sequences, whose
 * workspace grows with T); T == 1, T <= 12, float32, float16 and K = V = 128 take the
 * same kernels as in rwkv7_fwd, which need no workspace.  The call itself allocates
 * nothing and calls no allocating routine; its first call on a device looks the
 * array's address up (hipGetSymbolAddress), so make that one outside a capture.  All
 * calls on one GPU share the array: two of them that overlap in time (different
 * streams, or graphs replayed concurrently) race and give wrong results; calls on one
 * stream are ordered and safe.  Nothing in the array needs clearing between calls:
 * every launch marks the states it hands over with a fresh tag (see rwkv7_fwd_status). */
#define RWKV7_NOALLOC_MAX_BH 256
int rwkv7_fwd_noalloc(const void* r, const void* w, const void* k, const void* v,
                      const void* a, const void* b,
                      const float* h0, int64_t h0_batch_stride,
                      void* o, float* ht,
                      int B, int T, int H, int K, int V, int dtype, void* stream);

/* ---- did a chunked forward finish? ------------------------------------------------
 * The one-kernel chunked forward hands each (batch, head) state from one 64-token
 * chunk's workgroup to the next through the workspace; a workgroup waits for its
 * predecessor for at most two seconds (a chunk takes microseconds).  Should a wait
 * ever time out -- which no correct launch does -- the kernel still drains: the
 * waiting waves stop, fill what they would have written of o and ht with NaN, and
 * leave a mark in a 16-byte status record inside the workspace.  The call itself has
 * returned 0 long before, so this record is how a caller tells "the library gave
 * up" from "my inputs held NaN": after synchronising the stream ITSELF, copy the 16
 * bytes at  (char*)ws + rwkv7_fwd_status_offset(B, T, H, dtype)  to the host and
 * pass them to rwkv7_fwd_status().  The record belongs to the last forward that ran
 * with this workspace: rwkv7_fwd and rwkv7_fwd_gather (offset from
 * rwkv7_fwd_status_offset), rwkv7_fwd_varlen (rwkv7_fwd_varlen_status_offset), and the
 * two-kernel form, whose summary launch writes a record that can only read "done".
 * The offset functions return RWKV7_NO_STATUS_RECORD for shapes and dtypes whose call
 * runs no chunked kernel (T <= 12, float32, float16).  They take no head size: a call at K = V = 128
 * writes no record either (its kernels use no workspace), so do not ask for one there.  No counterpart in
 * the reference, whose kernels do not communicate. */
#define RWKV7_NO_STATUS_RECORD ((size_t)-1)
#define RWKV7_FWD_DONE      0   /* the launch that wrote the record did not give up */
#define RWKV7_FWD_GAVE_UP   1   /* a hand-off wait timed out: o and ht hold NaN */
#define RWKV7_FWD_NO_LAUNCH 2   /* the record is zero: no launch has written it */
size_t rwkv7_fwd_status_offset(int B, int T, int H, int dtype);
size_t rwkv7_fwd_varlen_status_offset(int n_seq, int T_total, int H, int dtype);
/* `record`: HOST pointer to a copy of the 16-byte record.  Returns RWKV7_FWD_* or RWKV7_ERR_NULL_POINTER. */
int rwkv7_fwd_status(const void* record);
/* The same news without a copy or a synchronisation: a word of pinned host memory that the device can write
 * (hipHostMalloc), set to 0 by the caller.  A one-kernel forward that gives up stores a non-zero value there
 * (besides its status record), which the host sees on a plain read some time after; a caller looks at the word
 * before its next call, say.  One word per process, NULL to take it away; the caller keeps the memory alive for
 * as long as it is registered.  No counterpart in the reference. */
int rwkv7_set_giveup_notice(unsigned long long* host_word);

/* ---- initial states gathered through a map -----------------------------------------
 * The reference's RWKV6 operator lets several batch rows start from one of a few
 * stored states: init_state [n_state, H, K, K] with state_map [B]
 * (/root/reference/rwkv_ops/rwkv6_kernel/ops_rwkv_kernel.py:37-57,
 * torch_rwkv_kernel.py:259-298: `ops.take(init_state, state_map, axis=0)`); its RWKV7
 * operator has no such argument.  These two calls give the RWKV7 path the same
 * facility without materialising the gathered states: batch row b starts from
 * states[state_map[b]] (float32 [n_state, H, 64, 64]; state_map int32 [B] on the
 * device; entries outside [0, n_state) are clamped so that a bad map cannot fault).
 * rwkv7_fwd_gather otherwise equals rwkv7_fwd (ht dense [B, H, 64, 64], nullable).
 * rwkv7_decode_step_gather: ht dense, or ht = NULL to write each row's new state
 * back into the slot it was read from (a state pool updated in place; the entries of
 * state_map must then be distinct). */
int rwkv7_fwd_gather(const void* r, const void* w, const void* k, const void* v,
                     const void* a, const void* b,
                     const float* states, int n_state, const int32_t* state_map,
                     void* o, float* ht,
                     int B, int T, int H, int K, int V, int dtype,
                     void* ws, size_t ws_bytes, void* stream);
int rwkv7_decode_step_gather(const void* r, const void* w, const void* k, const void* v,
                             const void* a, const void* b,
                             float* states, int n_state, const int32_t* state_map,
                             void* o, float* ht,
                             int B, int H, int K, int V, int dtype, void* stream);

/* The same bf16 forward as two kernels with the per-chunk summaries in HBM (the form
 * the backward pass builds on), for callers that want the halves separately.
 * rwkv7_fwd_chunk_summary replaces the chunk-parallel launches of chunk_dplr_fwd
 * (torch_op.py:81-98: cumsum, intra-chunk A, WY inverse, w/u) and fills ws;
 * rwkv7_fwd_chunk_scan replaces its serial scan and output launches
 * (torch_op.py:101-117) and consumes ws.  bf16 only (f32: RWKV7_ERR_UNSUPPORTED);
 * the same ws (rwkv7_fwd_chunk_workspace_bytes, 32.25 KiB per chunk and head, + 256 bytes
 * for the status record at offset rwkv7_fwd_chunk_workspace_bytes() - 256) must be passed to both. */
size_t rwkv7_fwd_chunk_workspace_bytes(int B, int T, int H, int dtype);
int rwkv7_fwd_chunk_summary(const void* r, const void* w, const void* k, const void* v,
                            const void* a, const void* b,
                            int B, int T, int H, int K, int V, int dtype,
                            void* ws, size_t ws_bytes, void* stream);
int rwkv7_fwd_chunk_scan(const float* h0, int64_t h0_batch_stride, void* o, float* ht,
                         int B, int T, int H, int K, int V, int dtype,
                         const void* ws, size_t ws_bytes, void* stream);

/* ---- backward over a sequence ---------------------------------------------------
 * Replaces ChunkDPLRDeltaRuleFunction.backward / chunk_dplr_bwd
 * (/root/reference/rwkv_ops/rwkv7_kernel/torch_op.py:123-265,304-325) together with
 * the autograd of the outer `-exp(w)` (:434): given the forward inputs, d_o (gradient
 * of o, [B,T,H,64], NULL = zero) and d_ht (gradient of the final state, float32
 * [B,H,64,64], NULL = zero), writes dr, dw, dk, dv, da, db ([B,T,H,64], `dtype`; dw is
 * the gradient with respect to the API's `w` argument) and, if dh0 != NULL, the
 * gradient of the initial state (float32 [B,H,64,64], one per batch entry even when
 * h0 is broadcast).  Forward intermediates are recomputed, nothing is saved by the
 * forward call.  bf16 runs the chunked MFMA backward; f32 (K = V = 64) beyond 12 tokens
 * runs the chunked float32 backward (16-token chunks on the float32 matrix cores: one more
 * forward pass that stores the state before every chunk, a kernel that walks the chain of
 * adjoint states per (batch, head), a kernel per (batch, head, chunk) for the rest; a call
 * in which some chunk's total decay is below e^-60 is done token by token instead, by the
 * kernel of rwkv7_bwd_recurrent, inside the same call), at most 12 tokens
 * rwkv7_bwd_recurrent below.  The float32 workspace is the larger one: 40 KiB per 16 tokens
 * and head plus 1 MiB per head (rwkv7_bwd_workspace_bytes answers for the dtype it is asked
 * about). */
size_t rwkv7_bwd_workspace_bytes(int B, int T, int H, int dtype);
int rwkv7_bwd(const void* r, const void* w, const void* k, const void* v,
              const void* a, const void* b,
              const float* h0, int64_t h0_batch_stride,
              const void* d_o, const float* d_ht,
              void* dr, void* dw, void* dk, void* dv, void* da, void* db, float* dh0,
              int B, int T, int H, int K, int V, int dtype,
              void* ws, size_t ws_bytes, void* stream);

/* The backward of the reference's native loop (native_keras_op.py:80-88, differentiated there by the host
 * framework's autograd) one token at a time in float32 arithmetic, for either dtype of the tensors
 * (bf16, f32, f16: values are widened on load, gradients rounded on store) and K = V = 64 or 128: the
 * token-by-token path -- head size 128, float16, float32 calls of a dozen tokens or with very strong decays --
 * two to three microseconds per token, not the throughput path.  Same arguments and meaning as rwkv7_bwd; dense
 * batches only.  The workspace (rwkv7_bwd_recurrent_workspace_bytes: the state of every (batch, head) at the start
 * of each 64-token segment (32 tokens for K = 128), plus one segment's worth of per-token states per (batch, head))
 * grows with B*H*T*K*V / 16.  K = 128 with at most 192 (batch, head) pairs splits the value columns of a head
 * over two workgroups and adds 40 bytes per element of a [B,T,H,K] tensor for their partial sums. */
size_t rwkv7_bwd_recurrent_workspace_bytes(int B, int T, int H, int K);
int rwkv7_bwd_recurrent(const void* r, const void* w, const void* k, const void* v,
                        const void* a, const void* b,
                        const float* h0, int64_t h0_batch_stride,
                        const void* d_o, const float* d_ht,
                        void* dr, void* dw, void* dk, void* dv, void* da, void* db, float* dh0,
                        int B, int T, int H, int K, int V, int dtype,
                        void* ws, size_t ws_bytes, void* stream);

/* ---- packed sequences of different lengths ------------------------------------------
 * The reference declares `cu_seqlens` on chunk_dplr_delta_rule and on its autograd node
 * (/root/reference/rwkv_ops/rwkv7_kernel/torch_op.py:283,338,363-365,388-398) with the
 * FlashAttention meaning -- the batch is ONE row of T_total tokens, sequence i is tokens
 * cu_seqlens[i] .. cu_seqlens[i+1]-1, one initial and one final state per sequence -- but
 * never hands it to its kernels (torch_op.py:286-297 drops it; the kernels' branches are
 * stripped, e.g. triton_kernel/chunk_h_fwd.py:51-58).  These calls implement that
 * meaning: r..b, o and the gradients are [T_total, H, 64]; cu_seqlens is int32
 * [n_seq + 1] on the device, starting at 0, non-decreasing, ending at T_total at most
 * (rows of o and of the gradients beyond the last entry are filled with zeros; values are
 * clamped into [0, T_total] on the device and a table whose spans overlap has the chunks
 * beyond T_total / 64 + n_seq dropped, so a bad table gives meaningless results, never a fault); h0, ht, d_ht
 * and dh0 are float32 [n_seq, H, 64, 64] (h0_batch_stride 0 broadcasts one state).  A
 * sequence may be empty: its final state is its initial state.  Chunks are counted from
 * each sequence's own first token, so the result for a sequence does not depend on
 * where it lies in the packed row.  The lengths never travel to the host: grids and
 * workspaces are sized for the most chunks T_total tokens in n_seq sequences can have
 * (T_total / 64 + n_seq per head).  bf16 and f32 (f32: the chunked float32 kernels on 16-token chunks,
 * T_total / 16 + n_seq records per head in the backward's workspace; the forward takes none). */
size_t rwkv7_fwd_varlen_workspace_bytes(int n_seq, int T_total, int H, int dtype);
int rwkv7_fwd_varlen(const void* r, const void* w, const void* k, const void* v,
                     const void* a, const void* b,
                     const int32_t* cu_seqlens, int n_seq,
                     const float* h0, int64_t h0_batch_stride,
                     void* o, float* ht,
                     int T_total, int H, int K, int V, int dtype,
                     void* ws, size_t ws_bytes, void* stream);
size_t rwkv7_bwd_varlen_workspace_bytes(int n_seq, int T_total, int H, int dtype);
int rwkv7_bwd_varlen(const void* r, const void* w, const void* k, const void* v,
                     const void* a, const void* b,
                     const int32_t* cu_seqlens, int n_seq,
                     const float* h0, int64_t h0_batch_stride,
                     const void* d_o, const float* d_ht,
                     void* dr, void* dw, void* dk, void* dv, void* da, void* db, float* dh0,
                     int T_total, int H, int K, int V, int dtype,
                     void* ws, size_t ws_bytes, void* stream);
/* rwkv7_bwd_recurrent over packed sequences: the token-by-token float32 backward (bf16, f32 or f16 tensors,
 * K = V = 64 or 128) with the arguments of rwkv7_bwd_varlen -- what rwkv7_bwd_varlen runs for packed rows at head
 * size 128.  No counterpart in the reference, like the packed calls above.  Workspace: one
 * state per segment of 64 tokens (32 at K = 128) for T_total / segment + n_seq segments per head, plus a segment's
 * worth of states for each of at most 1024 (sequence, head) pairs walked at a time. */
size_t rwkv7_bwd_recurrent_varlen_workspace_bytes(int n_seq, int T_total, int H, int K);
int rwkv7_bwd_recurrent_varlen(const void* r, const void* w, const void* k, const void* v,
                               const void* a, const void* b,
                               const int32_t* cu_seqlens, int n_seq,
                               const float* h0, int64_t h0_batch_stride,
                               const void* d_o, const float* d_ht,
                               void* dr, void* dw, void* dk, void* dv, void* da, void* db, float* dh0,
                               int T_total, int H, int K, int V, int dtype,
                               void* ws, size_t ws_bytes, void* stream);

/* The float32 recurrent kernel for either dtype (inputs are widened on load):
 * the arithmetic of native_keras_op.py:85,87 one token at a time with the state
 * in registers.  Slow; what float16 tensors, head size 128 in float32 and sequences of at most 12 tokens
 * run, and an on-device cross-check for the chunked kernels. */
int rwkv7_fwd_recurrent(const void* r, const void* w, const void* k, const void* v,
                        const void* a, const void* b,
                        const float* h0, int64_t h0_batch_stride,
                        void* o, float* ht,
                        int B, int T, int H, int K, int V, int dtype, void* stream);

/* ---- one decode step (T = 1) --------------------------------------------------
 * r..b and o are [B, H, 64].  Reads the state once and writes the new state once;
 * ht == h0 (in place) is allowed when h0_batch_stride != 0.  The reference has no
 * dedicated step: it pads T = 1 to a 16-token chunk and runs all six kernels
 * (torch_op.py:80); its arithmetic is one iteration of native_keras_op.py:80-88. */
int rwkv7_decode_step(const void* r, const void* w, const void* k, const void* v,
                      const void* a, const void* b,
                      const float* h0, int64_t h0_batch_stride,
                      void* o, float* ht,
                      int B, int H, int K, int V, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* RWKV7_MI355X_H */
