/* C ABI of the RWKV6 operator in librwkv7_mi355x.so (MI355X, gfx950): the same library, conventions and
 * status codes as include/rwkv7_mi355x.h (plain device pointers, nothing allocates or synchronises, the
 * kernels are enqueued on `stream`; 0 = ok, < 0 = RWKV7_ERR_*, > 0 = hipError_t).
 *
 * Operator (per batch b and head h, state s[K][V] float32, K = V = 64 or 128), as the reference's loop defines it
 * (/root/reference/rwkv_ops/rwkv6_kernel/ops_rwkv_kernel.py:59-73) and its GPU kernels compute it
 * (rwkv6_kernel/torch_kernel/wkv6_cuda.cu, rwkv6_kernel/jax_kernel_hip/rwkv_kernels.hip:114-163):
 *     d_t = exp(-exp(w_t))
 *     y_t = r_t^T (diag(u) k_t v_t^T + s_{t-1})
 *     s_t = k_t v_t^T + diag(d_t) s_{t-1}
 *
 * Replaces the kernels behind RWKVKernelOperator.__call__
 * (/root/reference/rwkv_ops/rwkv6_kernel/torch_rwkv_kernel.py:155-209,213-330: forward_{bf16,fp32} and
 * forward_with_state_{bf16,fp32}): r, k, v, w and y are [B, T, C] = [B, T, H, 64] contiguous in `dtype`,
 * u is [H, 64] in `dtype`.  Initial states are float32 [n_state, H, 64, 64] (key index first, as the
 * reference's kernels lay them out, rwkv_kernels.hip:180-196) gathered through state_map (int32 [B] on the
 * device, entries clamped into range): batch row b starts from states[state_map[b]]
 * (ops_rwkv_kernel.py:37-57).  state_map == NULL: n_state must be 1 (shared by all rows) or B (row b takes
 * state b).  states == NULL: zero states.  ys (nullable) receives the final states, float32 [B, H, 64, 64].
 *
 * bf16 with T > 1 runs the chunked MFMA kernels of the RWKV7 path in their RWKV6 mode and needs the
 * workspace of rwkv6_fwd_workspace_bytes(); T == 1 runs the decode kernel in its RWKV6 mode (the state is
 * read once and written once; ys == states updates a dense [B, H, 64, 64] state in place), float32 with
 * T > 1 the float32 recurrent kernel; neither needs a workspace.
 *
 * K = V = 128 (the reference builds its kernels for any head size, torch_rwkv_kernel.py:22-45: -D_N_): every
 * shape above with 128 in the place of 64.  T == 1 runs the decode kernel, longer sequences the float32
 * recurrent kernel for bf16 and float32 alike (there is no chunked RWKV6 kernel at this head size); no
 * workspace is read, ws may be NULL. */
#ifndef RWKV6_MI355X_H
#define RWKV6_MI355X_H

#include "rwkv7_mi355x.h"

#ifdef __cplusplus
extern "C" {
#endif

size_t rwkv6_fwd_workspace_bytes(int B, int T, int H, int dtype);
int rwkv6_fwd(const void* r, const void* k, const void* v, const void* w, const void* u,
              const float* states, int n_state, const int32_t* state_map,
              void* y, float* ys,
              int B, int T, int H, int K, int V, int dtype,
              void* ws, size_t ws_bytes, void* stream);

/* The float32 recurrent kernel for either dtype and any T: the accurate path and the on-device
 * cross-check of the chunked one.  Same arguments, no workspace. */
int rwkv6_fwd_recurrent(const void* r, const void* k, const void* v, const void* w, const void* u,
                        const float* states, int n_state, const int32_t* state_map,
                        void* y, float* ys,
                        int B, int T, int H, int K, int V, int dtype, void* stream);

/* ---- backward of the call without a state ---------------------------------------------------------
 * Replaces RWKV_6.backward (/root/reference/rwkv_ops/rwkv6_kernel/torch_rwkv_kernel.py:93-152: the four
 * backward kernels of wkv6_cuda.cu and the sum of gu over the batch): given r, k, v, w, u and d_y
 * ([B, T, H, 64], bf16 or float32), writes dr, dk, dv, dw (same shape and type; dw is the gradient with respect to the
 * w argument, the decay being exp(-exp(w))) and du (float32 [H, 64], already summed over the batch).  The
 * initial state is zero and no final state is returned, as in the reference's differentiable path.  The
 * state-path gradients come from the RWKV7 backward kernels run on the operands read one token ahead
 * (r_{t+1} against k_t, v_t, w_t); the bonus term's gradient is added by an epilogue kernel.  float32 tensors
 * run the float32 kernels and get float32-accurate gradients, as the reference's float32 kernel gives them
 * (torch_rwkv_kernel.py:137); float16: RWKV7_ERR_UNSUPPORTED.
 * K = V = 128: the state path is the float32 recurrent backward of the RWKV7 operator over the same operands, for
 * bf16 and float32 tensors; its workspace size comes from rwkv6_bwd_workspace_bytes_head(), which takes the head
 * size (rwkv6_bwd_workspace_bytes() is the K = V = 64 value). */
size_t rwkv6_bwd_workspace_bytes(int B, int T, int H, int dtype);
size_t rwkv6_bwd_workspace_bytes_head(int B, int T, int H, int K, int dtype);
int rwkv6_bwd(const void* r, const void* k, const void* v, const void* w, const void* u,
              const void* d_y,
              void* dr, void* dk, void* dv, void* dw, float* du,
              int B, int T, int H, int K, int V, int dtype,
              void* ws, size_t ws_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* RWKV6_MI355X_H */
