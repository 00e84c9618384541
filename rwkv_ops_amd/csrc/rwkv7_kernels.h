// Internal launch interface between the C ABI (rwkv7_api.hip) and the kernel files.
#pragma once

#include <atomic>

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "rwkv7_common.h"

namespace rwkv7 {

struct SeqArgs {
    const void *r, *w, *k, *v, *a, *b;
    const float* h0;          // nullable
    int64_t h0_batch_stride;  // 0 or H*64*64
    const int* h0_map;        // nullable: batch row b starts from state h0_map[b] (clamped to [0, n_state))
    int n_state;              // number of states behind h0 when h0_map is given
    bool ht_in_place;         // decode with a map: the new state goes back to the slot it was read from
    void* o;
    float* ht;                // nullable
    int B, T, H;
    int N;                    // head size K = V: 64, or 128 (decode and float32 recurrent kernels only)
    int dtype;                // RWKV7_DTYPE_*
    const int* cu;            // nullable: cumulative sequence lengths [B + 1] on the device; the tensors are
                              // then one packed row of T tokens in all and B counts the sequences
    const void* u6;           // nullable: not NULL selects the RWKV6 operator, u6 = its bonus [H, 64] (a, b unused)
};

hipError_t launch_decode(const SeqArgs& p, hipStream_t stream);
hipError_t launch_fwd_recurrent(const SeqArgs& p, hipStream_t stream);
// the RWKV6 operator one token at a time in float32 (p.u6 != NULL; p.a and p.b are not read)
hipError_t launch_rwkv6_recurrent(const SeqArgs& p, hipStream_t stream);

// chunked bf16 forward (T >= 1); ws must hold fwd_chunk_workspace_bytes(B, T, H) bytes, 256-byte aligned
size_t fwd_chunk_workspace_bytes(int B, int T, int H, bool varlen = false);
hipError_t launch_fwd_chunk(const SeqArgs& p, void* ws, hipStream_t stream);
// the same forward as ONE kernel: each chunk's workgroup applies its summary to the state it receives
// from the previous chunk's workgroup and hands the new state on (ws: fwd_fused_workspace_bytes)
size_t fwd_fused_workspace_bytes(int B, int T, int H, bool varlen = false);
// ... of which, for bh (batch, head) sequences: the status record padded to 256 bytes, two float32 state slots
// per sequence and head and the slots' 1 KiB carriers
constexpr size_t fwd_fused_bytes(size_t bh) { return 256 + 2 * bh * (4096 * 4 + 1024); }
// Byte offset, within the workspace of either form, of the launch's 16-byte status record (two 64-bit
// words): [1] = the launch's tag (never 0), [0] = that tag if a hand-off wait of the one-kernel form timed
// out and the outputs were poisoned, anything else otherwise.
size_t fwd_fused_status_offset(int B, int T, int H, bool varlen = false);
size_t fwd_chunk_status_offset(int B, int T, int H, bool varlen = false);
hipError_t launch_fwd_fused(const SeqArgs& p, void* ws, hipStream_t stream);
// the word (device-accessible host memory, or null) that a fused forward which gives up writes its tag into
std::atomic<unsigned long long*>& giveup_notice();
// its two halves: the parallel per-chunk summaries (reads r..b, fills ws) and the serial scan
// (reads ws and h0, writes o and ht)
hipError_t launch_fwd_chunk_summary(const SeqArgs& p, void* ws, hipStream_t stream);
hipError_t launch_fwd_chunk_scan(const SeqArgs& p, void* ws, hipStream_t stream);

// chunked bf16 forward for K = V = 128 (p.N == 128): no workspace; dense or packed (p.cu), state map honoured
hipError_t launch_fwd_chunk128(const SeqArgs& p, hipStream_t stream);

// chunked float32 forward (float32 tensors, K = V = 64) on the float32 matrix cores: no workspace; dense or packed
// (p.cu), state map honoured
hipError_t launch_fwd_chunk_f32(const SeqArgs& p, hipStream_t stream);
// the same kernel without outputs, storing the state at the start of every `seg` tokens ([B*H][ceil(T/seg)][64][64])
hipError_t launch_fwd_chunk_f32_states(const SeqArgs& p, float* states, int seg, hipStream_t stream, int* strong = nullptr);

struct BwdArgs {
    const void *r, *w, *k, *v, *a, *b;
    const float* h0;          // nullable
    int64_t h0_batch_stride;
    const void* dO;           // nullable (zero)
    const float* dht;         // nullable (zero)
    void *dr, *dw, *dk, *dv, *da, *db;
    float* dh0;               // nullable, [B, H, 64, 64]
    int B, T, H;
    int dtype;
    const int* cu;            // as in SeqArgs
};

// Packed sequences: the list of existing chunks that the chunked kernels launch over (first
// chunk_items_bytes of their workspace); also copies src -> dst for sequences without tokens.
// `tail`: up to six [T, H, 64] output tensors whose rows behind the last sequence are set to zero.
struct TailFill { void* p[6]; int n; int64_t row_bytes; };
size_t chunk_items_bytes(int B, int T);
SeqLayout seq_layout(const SeqArgs& p, const void* ws);
TailFill tail_of_output(const SeqArgs& p);
hipError_t launch_chunk_items(const SeqLayout& L, void* items, const float* src, int64_t src_batch_stride,
                              float* dst, const TailFill& tail, hipStream_t stream);

// chunked bf16 backward; ws must hold bwd_chunk_workspace_bytes(B, T, H) bytes, 256-byte aligned
size_t bwd_chunk_workspace_bytes(int B, int T, int H, bool varlen = false);
hipError_t launch_bwd_chunk(const BwdArgs& p, void* ws, hipStream_t stream);
// float32 recurrent backward for any dtype, K = V = N in {64, 128}, dense batches or packed sequences (p.cu):
// ws holds bwd_recurrent_workspace_bytes(B, T, H, N) bytes (segment states, then per-workgroup scratch)
size_t bwd_recurrent_workspace_bytes(int B, int T, int H, int N, bool varlen = false);
hipError_t launch_bwd_recurrent(const BwdArgs& p, int N, void* ws, hipStream_t stream);
hipError_t launch_fwd_recurrent_states(const SeqArgs& p, float* states, int seg, hipStream_t stream);
// its second launch alone, float32 tensors at K = V = 64, over states stored every 16 tokens; runs only when one of
// the n_flags integers at run_if_any is not zero
constexpr int WALK_MAX_GRID = 1024;     // workgroups of the walk over packed sequences (each owns 1 MiB of scratch)
hipError_t launch_bwd_recurrent_walk_f32(const BwdArgs& p, const float* states16, float* scratch,
                                         const int* run_if_any, int n_flags, hipStream_t stream);
// chunked float32 backward (float32 tensors, K = V = 64; dense batches or packed sequences, p.cu) on the float32 matrix cores;
// ws holds bwd_chunk_f32_workspace_bytes(B, T, H) bytes, 256-byte aligned
size_t bwd_chunk_f32_workspace_bytes(int B, int T, int H, bool varlen = false);
hipError_t launch_bwd_chunk_f32(const BwdArgs& p, void* ws, hipStream_t stream);
// RWKV6 backward (stateless call, bf16 or float32): runs the RWKV7 backward kernels on operands read one token ahead
// plus an epilogue for the bonus term; du is float32 [H, 64]
size_t rwkv6_bwd_workspace_bytes(int B, int T, int H, int N, int dtype);
hipError_t launch_rwkv6_bwd(const void* r, const void* k, const void* v, const void* w, const void* u,
                            const void* dy, void* dr, void* dk, void* dv, void* dw, float* du,
                            int B, int T, int H, int N, int dtype, void* ws, hipStream_t stream);
// the backward's variant of the chunk summaries (rwkv7_fwd_chunk.hip)
hipError_t launch_bwd_summary(const SeqArgs& p, const SeqLayout& L, const void* d_o, void* qdo, void* pp,
                              void* qc, float* eg, hipStream_t stream);

}  // namespace rwkv7
