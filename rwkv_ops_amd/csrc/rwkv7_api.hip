// extern "C" entry points of librwkv7_mi355x.so: argument validation, then launch.
// Nothing here allocates or synchronises.
#include "../../include/rwkv7_mi355x.h"
#include "../../include/rwkv6_mi355x.h"
#include "rwkv7_kernels.h"

#include <atomic>

using rwkv7::SeqArgs;

namespace {

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// wide_ok: the entry point also has kernels for K = V = 128
int check_seq(const void* r, const void* w, const void* k, const void* v, const void* a,
              const void* b, const float* h0, int64_t h0_batch_stride, const void* o,
              const float* ht, int B, int T, int H, int K, int V, int dtype, bool wide_ok = false,
              bool half_ok = false)
{
    // half_ok: the entry point reaches the decode step or the recurrent forward, which also read float16
    if (dtype == RWKV7_DTYPE_F16) { if (!half_ok) return RWKV7_ERR_UNSUPPORTED; }
    else if (dtype != RWKV7_DTYPE_BF16 && dtype != RWKV7_DTYPE_F32) return RWKV7_ERR_BAD_DTYPE;
    if (K != V || (K != 64 && !(wide_ok && K == 128))) return RWKV7_ERR_BAD_HEAD_SIZE;
    if (B < 1 || T < 1 || H < 1) return RWKV7_ERR_BAD_SHAPE;
    // element offsets are 64-bit in the kernels; grids are 32-bit in (B*H) and (B*H*chunks)
    if ((int64_t)B * H > (int64_t)1 << 30) return RWKV7_ERR_BAD_SHAPE;
    if ((int64_t)B * H * ((T + 63) / 64) > (int64_t)1 << 30) return RWKV7_ERR_BAD_SHAPE;
    if (!r || !w || !k || !v || !a || !b || !o) return RWKV7_ERR_NULL_POINTER;
    if (h0 && h0_batch_stride != 0 && h0_batch_stride != (int64_t)H * K * V)
        return RWKV7_ERR_BAD_STRIDE;
    if (!aligned16(r) || !aligned16(w) || !aligned16(k) || !aligned16(v) || !aligned16(a) ||
        !aligned16(b) || !aligned16(o) || !aligned16(h0) || !aligned16(ht))
        return RWKV7_ERR_ALIGNMENT;
    return RWKV7_OK;
}

SeqArgs pack(const void* r, const void* w, const void* k, const void* v, const void* a,
             const void* b, const float* h0, int64_t h0_batch_stride, void* o, float* ht,
             int B, int T, int H, int dtype, int N = 64)
{
    SeqArgs p;
    p.N = N;
    p.r = r; p.w = w; p.k = k; p.v = v; p.a = a; p.b = b;
    p.h0 = h0; p.h0_batch_stride = h0 ? h0_batch_stride : 0;
    p.h0_map = nullptr; p.n_state = 0; p.ht_in_place = false;
    p.o = o; p.ht = ht; p.B = B; p.T = T; p.H = H; p.dtype = dtype; p.cu = nullptr; p.u6 = nullptr;
    return p;
}

}  // namespace

extern "C" {

int rwkv7_abi_version(void) { return RWKV7_ABI_VERSION; }

const char* rwkv7_status_string(int status) {
    switch (status) {
        case RWKV7_OK: return "ok";
        case RWKV7_ERR_NULL_POINTER: return "a required pointer is NULL";
        case RWKV7_ERR_BAD_DTYPE: return "dtype must be RWKV7_DTYPE_BF16 (0), RWKV7_DTYPE_F32 (1) or RWKV7_DTYPE_F16 (2)";
        case RWKV7_ERR_BAD_HEAD_SIZE: return "K = V = 64 (every entry point) or 128 (every entry point but the two-kernel ones) only";
        case RWKV7_ERR_BAD_SHAPE: return "B, T and H must be >= 1 and B*H*ceil(T/64) <= 2^30";
        case RWKV7_ERR_BAD_STRIDE: return "h0_batch_stride must be 0 (broadcast) or H*K*V";
        case RWKV7_ERR_WORKSPACE: return "workspace is NULL, not 256-byte aligned or too small";
        case RWKV7_ERR_ALIGNMENT: return "tensor pointers must be 16-byte aligned";
        case RWKV7_ERR_UNSUPPORTED: return "this combination of arguments is not built";
        case RWKV7_ERR_TOO_LARGE: return "rwkv7_fwd_noalloc: B*H exceeds RWKV7_NOALLOC_MAX_BH (256), the size of the library's static scratch";
        default: break;
    }
    if (status > 0) return hipGetErrorString(static_cast<hipError_t>(status));
    return "unknown rwkv7 status";
}

int rwkv7_decode_step(const void* r, const void* w, const void* k, const void* v, const void* a,
                      const void* b, const float* h0, int64_t h0_batch_stride, void* o, float* ht,
                      int B, int H, int K, int V, int dtype, void* stream)
{
    int rc = check_seq(r, w, k, v, a, b, h0, h0_batch_stride, o, ht, B, 1, H, K, V, dtype, true, true);
    if (rc != RWKV7_OK) return rc;
    if (h0 && h0 == ht && h0_batch_stride == 0 && B > 1) return RWKV7_ERR_BAD_STRIDE;
    return (int)rwkv7::launch_decode(pack(r, w, k, v, a, b, h0, h0_batch_stride, o, ht, B, 1, H, dtype, K),
                                     static_cast<hipStream_t>(stream));
}

int rwkv7_fwd_recurrent(const void* r, const void* w, const void* k, const void* v, const void* a,
                        const void* b, const float* h0, int64_t h0_batch_stride, void* o, float* ht,
                        int B, int T, int H, int K, int V, int dtype, void* stream)
{
    int rc = check_seq(r, w, k, v, a, b, h0, h0_batch_stride, o, ht, B, T, H, K, V, dtype, true, true);
    if (rc != RWKV7_OK) return rc;
    return (int)rwkv7::launch_fwd_recurrent(
        pack(r, w, k, v, a, b, h0, h0_batch_stride, o, ht, B, T, H, dtype, K),
        static_cast<hipStream_t>(stream));
}

namespace {
// The one-kernel forward keeps a few chunks of every (batch, head) in flight, which pays when there are
// enough sequences to fill the chip; with few, long sequences the chain of state hand-offs is the
// critical path and the two-kernel form (parallel summaries, then a scan) is faster.
// (measured at T = 4096: 64 sequences 114 us against 140 us fused, 72 sequences 168 us against 150 us,
// 96 sequences 216 us against 179 us; at T = 16384: 64 sequences 472 us against 665 us, 80 sequences 777 us
// against 684 us)
bool use_fused_forward(int B, int H) { return (int64_t)B * H >= 72; }
// A handful of tokens per sequence (speculative-decoding verification, very short prompts) is faster one
// token at a time with the state in registers than through the 64-token chunk machinery, whatever the
// number of sequences: B*H = 2560, T = 2 / 8 / 16 / 32: 17 / 30 / 49 / 89 us against 46 / 46 / 47 / 49 us
// chunked; B*H = 40: 3.6 / 5.9 / 8.9 / 16 against 10 us.
constexpr int RECURRENT_MAX_T = 12;
// K = V = 128 in bf16 beyond that length: the chunked kernel for that head size (one workgroup per sequence and
// head, state in registers, no workspace)
bool takes_chunk128(const SeqArgs& p) { return p.N == 128 && p.dtype == RWKV7_DTYPE_BF16 && p.T > RECURRENT_MAX_T; }
// float32 tensors at K = V = 64 beyond that length: the chunked float32 kernel (16-token chunks on the float32 matrix
// cores, state in registers, no workspace)
bool takes_chunk_f32(const SeqArgs& p) { return p.N == 64 && p.dtype == RWKV7_DTYPE_F32 && p.T > RECURRENT_MAX_T; }
}  // namespace

size_t rwkv7_fwd_workspace_bytes(int B, int T, int H, int dtype) {
    if (dtype != RWKV7_DTYPE_BF16 || B < 1 || T < 2 || H < 1) return 0;
    return use_fused_forward(B, H) ? rwkv7::fwd_fused_workspace_bytes(B, T, H)
                                   : rwkv7::fwd_chunk_workspace_bytes(B, T, H);
}

size_t rwkv7_fwd_status_offset(int B, int T, int H, int dtype) {
    if (dtype != RWKV7_DTYPE_BF16 || B < 1 || T <= RECURRENT_MAX_T || H < 1) return RWKV7_NO_STATUS_RECORD;
    return use_fused_forward(B, H) ? rwkv7::fwd_fused_status_offset(B, T, H)
                                   : rwkv7::fwd_chunk_status_offset(B, T, H);
}

int rwkv7_set_giveup_notice(unsigned long long* host_word) {
    rwkv7::giveup_notice().store(host_word, std::memory_order_release);
    return RWKV7_OK;
}

int rwkv7_fwd_status(const void* record) {
    if (!record) return RWKV7_ERR_NULL_POINTER;
    const unsigned long long* rec = static_cast<const unsigned long long*>(record);
    if (rec[1] == 0ull) return RWKV7_FWD_NO_LAUNCH;
    return rec[0] == rec[1] ? RWKV7_FWD_GAVE_UP : RWKV7_FWD_DONE;
}

size_t rwkv7_fwd_chunk_workspace_bytes(int B, int T, int H, int dtype) {
    if (dtype != RWKV7_DTYPE_BF16 || B < 1 || T < 1 || H < 1) return 0;
    return rwkv7::fwd_chunk_workspace_bytes(B, T, H);
}

int rwkv7_fwd(const void* r, const void* w, const void* k, const void* v, const void* a,
              const void* b, const float* h0, int64_t h0_batch_stride, void* o, float* ht,
              int B, int T, int H, int K, int V, int dtype, void* ws, size_t ws_bytes, void* stream)
{
    int rc = check_seq(r, w, k, v, a, b, h0, h0_batch_stride, o, ht, B, T, H, K, V, dtype, true, true);
    if (rc != RWKV7_OK) return rc;
    SeqArgs p = pack(r, w, k, v, a, b, h0, h0_batch_stride, o, ht, B, T, H, dtype, K);
    if (T == 1) return (int)rwkv7::launch_decode(p, static_cast<hipStream_t>(stream));
    if (takes_chunk128(p)) return (int)rwkv7::launch_fwd_chunk128(p, static_cast<hipStream_t>(stream));
    if (takes_chunk_f32(p)) return (int)rwkv7::launch_fwd_chunk_f32(p, static_cast<hipStream_t>(stream));
    if (dtype != RWKV7_DTYPE_BF16 || K == 128 || T <= RECURRENT_MAX_T)   // the chunked kernels are K = V = 64 only
        return (int)rwkv7::launch_fwd_recurrent(p, static_cast<hipStream_t>(stream));
    const size_t need = rwkv7_fwd_workspace_bytes(B, T, H, dtype);
    if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return RWKV7_ERR_WORKSPACE;
    if (use_fused_forward(B, H)) return (int)rwkv7::launch_fwd_fused(p, ws, static_cast<hipStream_t>(stream));
    return (int)rwkv7::launch_fwd_chunk(p, ws, static_cast<hipStream_t>(stream));
}

/* ---- the forward for callers that may not allocate -------------------------------------------- */
namespace {
// The one-kernel forward's workspace (status record, two state slots per (batch, head) and their carriers)
// for RWKV7_NOALLOC_MAX_BH sequences, held by every GPU the library is loaded on until the process ends.
constexpr size_t SCRATCH_BYTES = rwkv7::fwd_fused_bytes(RWKV7_NOALLOC_MAX_BH);
static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];
// The array's name is a host-side stand-in; its device address differs per GPU and is looked up once per
// device (with that device current) and kept here.
constexpr int MAX_DEVICES = 64;
std::atomic<void*> scratch_ptr[MAX_DEVICES];

int scratch_on_current_device(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= MAX_DEVICES) return RWKV7_ERR_UNSUPPORTED;
    void* p = scratch_ptr[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (p == nullptr || (reinterpret_cast<uintptr_t>(p) & 255u) != 0) return RWKV7_ERR_WORKSPACE;
        scratch_ptr[dev].store(p, std::memory_order_release);    // (two threads racing here store the same address)
    }
    *out = p;
    return RWKV7_OK;
}
}  // namespace

int rwkv7_fwd_noalloc(const void* r, const void* w, const void* k, const void* v, const void* a,
                      const void* b, const float* h0, int64_t h0_batch_stride, void* o, float* ht,
                      int B, int T, int H, int K, int V, int dtype, void* stream)
{
    int rc = check_seq(r, w, k, v, a, b, h0, h0_batch_stride, o, ht, B, T, H, K, V, dtype, true, true);
    if (rc != RWKV7_OK) return rc;
    SeqArgs p = pack(r, w, k, v, a, b, h0, h0_batch_stride, o, ht, B, T, H, dtype, K);
    // the same routing as rwkv7_fwd for the kernels that use no workspace
    if (T == 1) return (int)rwkv7::launch_decode(p, static_cast<hipStream_t>(stream));
    if (takes_chunk128(p)) return (int)rwkv7::launch_fwd_chunk128(p, static_cast<hipStream_t>(stream));
    if (takes_chunk_f32(p)) return (int)rwkv7::launch_fwd_chunk_f32(p, static_cast<hipStream_t>(stream));
    if (dtype != RWKV7_DTYPE_BF16 || K == 128 || T <= RECURRENT_MAX_T)
        return (int)rwkv7::launch_fwd_recurrent(p, static_cast<hipStream_t>(stream));
    // Always the one-kernel form: its workspace does not grow with T.
    if ((int64_t)B * H > RWKV7_NOALLOC_MAX_BH || rwkv7::fwd_fused_workspace_bytes(B, T, H) > SCRATCH_BYTES)
        return RWKV7_ERR_TOO_LARGE;
    void* ws = nullptr;
    rc = scratch_on_current_device(&ws);
    if (rc != RWKV7_OK) return rc;
    return (int)rwkv7::launch_fwd_fused(p, ws, static_cast<hipStream_t>(stream));
}

/* ---- the same two calls with the initial states gathered through a map --------------------------- */
int rwkv7_fwd_gather(const void* r, const void* w, const void* k, const void* v, const void* a,
                     const void* b, const float* states, int n_state, const int32_t* state_map,
                     void* o, float* ht, int B, int T, int H, int K, int V, int dtype,
                     void* ws, size_t ws_bytes, void* stream)
{
    if (!states || !state_map) return RWKV7_ERR_NULL_POINTER;
    if (n_state < 1) return RWKV7_ERR_BAD_SHAPE;
    int rc = check_seq(r, w, k, v, a, b, states, (int64_t)H * K * V, o, ht, B, T, H, K, V, dtype, true, true);
    if (rc != RWKV7_OK) return rc;
    if ((reinterpret_cast<uintptr_t>(state_map) & 3u) != 0) return RWKV7_ERR_ALIGNMENT;
    SeqArgs p = pack(r, w, k, v, a, b, states, (int64_t)H * K * V, o, ht, B, T, H, dtype, K);
    p.h0_map = state_map; p.n_state = n_state;
    if (T == 1) return (int)rwkv7::launch_decode(p, static_cast<hipStream_t>(stream));
    if (takes_chunk128(p)) return (int)rwkv7::launch_fwd_chunk128(p, static_cast<hipStream_t>(stream));
    if (takes_chunk_f32(p)) return (int)rwkv7::launch_fwd_chunk_f32(p, static_cast<hipStream_t>(stream));
    if (dtype != RWKV7_DTYPE_BF16 || K == 128 || T <= RECURRENT_MAX_T)
        return (int)rwkv7::launch_fwd_recurrent(p, static_cast<hipStream_t>(stream));
    const size_t need = rwkv7_fwd_workspace_bytes(B, T, H, dtype);
    if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return RWKV7_ERR_WORKSPACE;
    if (use_fused_forward(B, H)) return (int)rwkv7::launch_fwd_fused(p, ws, static_cast<hipStream_t>(stream));
    return (int)rwkv7::launch_fwd_chunk(p, ws, static_cast<hipStream_t>(stream));
}

int rwkv7_decode_step_gather(const void* r, const void* w, const void* k, const void* v, const void* a,
                             const void* b, float* states, int n_state, const int32_t* state_map,
                             void* o, float* ht, int B, int H, int K, int V, int dtype, void* stream)
{
    if (!states || !state_map) return RWKV7_ERR_NULL_POINTER;
    if (n_state < 1) return RWKV7_ERR_BAD_SHAPE;
    int rc = check_seq(r, w, k, v, a, b, states, (int64_t)H * K * V, o, ht, B, 1, H, K, V, dtype, true, true);
    if (rc != RWKV7_OK) return rc;
    if ((reinterpret_cast<uintptr_t>(state_map) & 3u) != 0) return RWKV7_ERR_ALIGNMENT;
    SeqArgs p = pack(r, w, k, v, a, b, states, (int64_t)H * K * V, o, ht, B, 1, H, dtype, K);
    p.h0_map = state_map; p.n_state = n_state;
    p.ht_in_place = ht == nullptr;
    return (int)rwkv7::launch_decode(p, static_cast<hipStream_t>(stream));
}

int rwkv7_fwd_chunk_summary(const void* r, const void* w, const void* k, const void* v, const void* a,
                            const void* b, int B, int T, int H, int K, int V, int dtype,
                            void* ws, size_t ws_bytes, void* stream)
{
    if (dtype != RWKV7_DTYPE_BF16) return dtype == RWKV7_DTYPE_F32 || dtype == RWKV7_DTYPE_F16 ? RWKV7_ERR_UNSUPPORTED : RWKV7_ERR_BAD_DTYPE;
    int rc = check_seq(r, w, k, v, a, b, nullptr, 0, ws, nullptr, B, T, H, K, V, dtype);
    if (rc != RWKV7_OK) return rc;
    if (!ws || ws_bytes < rwkv7::fwd_chunk_workspace_bytes(B, T, H) || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0)
        return RWKV7_ERR_WORKSPACE;
    return (int)rwkv7::launch_fwd_chunk_summary(pack(r, w, k, v, a, b, nullptr, 0, nullptr, nullptr, B, T, H, dtype),
                                                ws, static_cast<hipStream_t>(stream));
}

int rwkv7_fwd_chunk_scan(const float* h0, int64_t h0_batch_stride, void* o, float* ht,
                         int B, int T, int H, int K, int V, int dtype,
                         const void* ws, size_t ws_bytes, void* stream)
{
    if (dtype != RWKV7_DTYPE_BF16) return dtype == RWKV7_DTYPE_F32 || dtype == RWKV7_DTYPE_F16 ? RWKV7_ERR_UNSUPPORTED : RWKV7_ERR_BAD_DTYPE;
    int rc = check_seq(ws, ws, ws, ws, ws, ws, h0, h0_batch_stride, o, ht, B, T, H, K, V, dtype);
    if (rc != RWKV7_OK) return rc == RWKV7_ERR_NULL_POINTER && !ws ? RWKV7_ERR_WORKSPACE : rc;
    if (ws_bytes < rwkv7::fwd_chunk_workspace_bytes(B, T, H) || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0)
        return RWKV7_ERR_WORKSPACE;
    return (int)rwkv7::launch_fwd_chunk_scan(
        pack(nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, h0, h0_batch_stride, o, ht, B, T, H, dtype),
        const_cast<void*>(ws), static_cast<hipStream_t>(stream));
}

size_t rwkv7_bwd_workspace_bytes(int B, int T, int H, int dtype) {
    if (B < 1 || T < 1 || H < 1) return 0;
    if (dtype == RWKV7_DTYPE_F32)
        return T > RECURRENT_MAX_T ? rwkv7::bwd_chunk_f32_workspace_bytes(B, T, H)
                                   : rwkv7::bwd_recurrent_workspace_bytes(B, T, H, 64);
    if (dtype != RWKV7_DTYPE_BF16) return 0;
    return rwkv7::bwd_chunk_workspace_bytes(B, T, H);
}

size_t rwkv7_bwd_recurrent_workspace_bytes(int B, int T, int H, int K) {
    if (B < 1 || T < 1 || H < 1 || (K != 64 && K != 128)) return 0;
    return rwkv7::bwd_recurrent_workspace_bytes(B, T, H, K);
}

int rwkv7_bwd_recurrent(const void* r, const void* w, const void* k, const void* v, const void* a, const void* b,
                        const float* h0, int64_t h0_batch_stride, const void* d_o, const float* d_ht,
                        void* dr, void* dw, void* dk, void* dv, void* da, void* db, float* dh0,
                        int B, int T, int H, int K, int V, int dtype, void* ws, size_t ws_bytes, void* stream)
{
    int rc = check_seq(r, w, k, v, a, b, h0, h0_batch_stride, dr, nullptr, B, T, H, K, V, dtype, true, true);
    if (rc != RWKV7_OK) return rc;
    if (!dw || !dk || !dv || !da || !db) return RWKV7_ERR_NULL_POINTER;
    if (!aligned16(d_o) || !aligned16(d_ht) || !aligned16(dw) || !aligned16(dk) || !aligned16(dv) ||
        !aligned16(da) || !aligned16(db) || !aligned16(dh0))
        return RWKV7_ERR_ALIGNMENT;
    const size_t need = rwkv7::bwd_recurrent_workspace_bytes(B, T, H, K);
    if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return RWKV7_ERR_WORKSPACE;
    rwkv7::BwdArgs p;
    p.r = r; p.w = w; p.k = k; p.v = v; p.a = a; p.b = b;
    p.h0 = h0; p.h0_batch_stride = h0 ? h0_batch_stride : 0;
    p.dO = d_o; p.dht = d_ht;
    p.dr = dr; p.dw = dw; p.dk = dk; p.dv = dv; p.da = da; p.db = db; p.dh0 = dh0;
    p.B = B; p.T = T; p.H = H; p.dtype = dtype; p.cu = nullptr;
    return (int)rwkv7::launch_bwd_recurrent(p, K, ws, static_cast<hipStream_t>(stream));
}

int rwkv7_bwd(const void* r, const void* w, const void* k, const void* v, const void* a, const void* b,
              const float* h0, int64_t h0_batch_stride, const void* d_o, const float* d_ht,
              void* dr, void* dw, void* dk, void* dv, void* da, void* db, float* dh0,
              int B, int T, int H, int K, int V, int dtype, void* ws, size_t ws_bytes, void* stream)
{
    // head size 128 has the token-by-token backward only (every dtype; its own workspace size)
    if (K == 128 && V == 128)
        return rwkv7_bwd_recurrent(r, w, k, v, a, b, h0, h0_batch_stride, d_o, d_ht, dr, dw, dk, dv, da, db, dh0,
                                   B, T, H, K, V, dtype, ws, ws_bytes, stream);
    // float32 gradients at K = V = 64: beyond a dozen tokens the chunked float32 backward, otherwise the
    // token-by-token one
    if (dtype == RWKV7_DTYPE_F32 && K == 64 && V == 64) {
        if (T <= RECURRENT_MAX_T)
            return rwkv7_bwd_recurrent(r, w, k, v, a, b, h0, h0_batch_stride, d_o, d_ht, dr, dw, dk, dv, da, db, dh0,
                                       B, T, H, K, V, dtype, ws, ws_bytes, stream);
        int rc = check_seq(r, w, k, v, a, b, h0, h0_batch_stride, dr, nullptr, B, T, H, K, V, dtype, true, true);
        if (rc != RWKV7_OK) return rc;
        if (!dw || !dk || !dv || !da || !db) return RWKV7_ERR_NULL_POINTER;
        if (!aligned16(d_o) || !aligned16(d_ht) || !aligned16(dw) || !aligned16(dk) || !aligned16(dv) ||
            !aligned16(da) || !aligned16(db) || !aligned16(dh0))
            return RWKV7_ERR_ALIGNMENT;
        const size_t need = rwkv7::bwd_chunk_f32_workspace_bytes(B, T, H);
        if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return RWKV7_ERR_WORKSPACE;
        rwkv7::BwdArgs p;
        p.r = r; p.w = w; p.k = k; p.v = v; p.a = a; p.b = b;
        p.h0 = h0; p.h0_batch_stride = h0 ? h0_batch_stride : 0;
        p.dO = d_o; p.dht = d_ht;
        p.dr = dr; p.dw = dw; p.dk = dk; p.dv = dv; p.da = da; p.db = db; p.dh0 = dh0;
        p.B = B; p.T = T; p.H = H; p.dtype = dtype; p.cu = nullptr;
        return (int)rwkv7::launch_bwd_chunk_f32(p, ws, static_cast<hipStream_t>(stream));
    }
    int rc = check_seq(r, w, k, v, a, b, h0, h0_batch_stride, dr, nullptr, B, T, H, K, V, dtype);
    if (rc != RWKV7_OK) return rc;
    if (!dw || !dk || !dv || !da || !db) return RWKV7_ERR_NULL_POINTER;
    if (!aligned16(d_o) || !aligned16(d_ht) || !aligned16(dw) || !aligned16(dk) || !aligned16(dv) ||
        !aligned16(da) || !aligned16(db) || !aligned16(dh0))
        return RWKV7_ERR_ALIGNMENT;
    const size_t need = rwkv7::bwd_chunk_workspace_bytes(B, T, H);
    if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return RWKV7_ERR_WORKSPACE;
    rwkv7::BwdArgs p;
    p.r = r; p.w = w; p.k = k; p.v = v; p.a = a; p.b = b;
    p.h0 = h0; p.h0_batch_stride = h0 ? h0_batch_stride : 0;
    p.dO = d_o; p.dht = d_ht;
    p.dr = dr; p.dw = dw; p.dk = dk; p.dv = dv; p.da = da; p.db = db; p.dh0 = dh0;
    p.B = B; p.T = T; p.H = H; p.dtype = dtype; p.cu = nullptr;
    return (int)rwkv7::launch_bwd_chunk(p, ws, static_cast<hipStream_t>(stream));
}

/* ---- packed sequences -------------------------------------------------------------------------- */
namespace {
int check_varlen(const int32_t* cu, int n_seq, int T_total, int H) {
    if (!cu) return RWKV7_ERR_NULL_POINTER;
    if ((reinterpret_cast<uintptr_t>(cu) & 3u) != 0) return RWKV7_ERR_ALIGNMENT;
    // the kernels launch over (T_total / 64 + n_seq) * H chunks at most
    if (n_seq < 1 || ((int64_t)(T_total >> 6) + n_seq) * H > (int64_t)1 << 30) return RWKV7_ERR_BAD_SHAPE;
    return RWKV7_OK;
}
}  // namespace

size_t rwkv7_fwd_varlen_workspace_bytes(int n_seq, int T_total, int H, int dtype) {
    if (dtype != RWKV7_DTYPE_BF16 || n_seq < 1 || T_total < 1 || H < 1) return 0;
    return use_fused_forward(n_seq, H) ? rwkv7::fwd_fused_workspace_bytes(n_seq, T_total, H, true)
                                       : rwkv7::fwd_chunk_workspace_bytes(n_seq, T_total, H, true);
}

size_t rwkv7_fwd_varlen_status_offset(int n_seq, int T_total, int H, int dtype) {
    if (dtype != RWKV7_DTYPE_BF16 || n_seq < 1 || T_total < 1 || H < 1) return RWKV7_NO_STATUS_RECORD;
    return use_fused_forward(n_seq, H) ? rwkv7::fwd_fused_status_offset(n_seq, T_total, H, true)
                                       : rwkv7::fwd_chunk_status_offset(n_seq, T_total, H, true);
}

int rwkv7_fwd_varlen(const void* r, const void* w, const void* k, const void* v, const void* a,
                     const void* b, const int32_t* cu_seqlens, int n_seq,
                     const float* h0, int64_t h0_batch_stride, void* o, float* ht,
                     int T_total, int H, int K, int V, int dtype, void* ws, size_t ws_bytes, void* stream)
{
    int rc = check_seq(r, w, k, v, a, b, h0, h0_batch_stride, o, ht, 1, T_total, H, K, V, dtype, true, true);
    if (rc != RWKV7_OK) return rc;
    rc = check_varlen(cu_seqlens, n_seq, T_total, H);
    if (rc != RWKV7_OK) return rc;
    SeqArgs p = pack(r, w, k, v, a, b, h0, h0_batch_stride, o, ht, n_seq, T_total, H, dtype, K);
    p.cu = cu_seqlens;
    if (takes_chunk128(p)) return (int)rwkv7::launch_fwd_chunk128(p, static_cast<hipStream_t>(stream));
    if (takes_chunk_f32(p)) return (int)rwkv7::launch_fwd_chunk_f32(p, static_cast<hipStream_t>(stream));
    if (dtype != RWKV7_DTYPE_BF16 || K == 128)
        return (int)rwkv7::launch_fwd_recurrent(p, static_cast<hipStream_t>(stream));
    const size_t need = rwkv7_fwd_varlen_workspace_bytes(n_seq, T_total, H, dtype);
    if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return RWKV7_ERR_WORKSPACE;
    if (use_fused_forward(n_seq, H)) return (int)rwkv7::launch_fwd_fused(p, ws, static_cast<hipStream_t>(stream));
    return (int)rwkv7::launch_fwd_chunk(p, ws, static_cast<hipStream_t>(stream));
}

size_t rwkv7_bwd_varlen_workspace_bytes(int n_seq, int T_total, int H, int dtype) {
    if (n_seq < 1 || T_total < 1 || H < 1) return 0;
    if (dtype == RWKV7_DTYPE_F32) return rwkv7::bwd_chunk_f32_workspace_bytes(n_seq, T_total, H, true);
    if (dtype != RWKV7_DTYPE_BF16) return 0;
    return rwkv7::bwd_chunk_workspace_bytes(n_seq, T_total, H, true);
}

int rwkv7_bwd_varlen(const void* r, const void* w, const void* k, const void* v, const void* a, const void* b,
                     const int32_t* cu_seqlens, int n_seq, const float* h0, int64_t h0_batch_stride,
                     const void* d_o, const float* d_ht,
                     void* dr, void* dw, void* dk, void* dv, void* da, void* db, float* dh0,
                     int T_total, int H, int K, int V, int dtype, void* ws, size_t ws_bytes, void* stream)
{
    if (K == 128 && V == 128)           // head size 128: the token-by-token backward (its own workspace size)
        return rwkv7_bwd_recurrent_varlen(r, w, k, v, a, b, cu_seqlens, n_seq, h0, h0_batch_stride, d_o, d_ht,
                                          dr, dw, dk, dv, da, db, dh0, T_total, H, K, V, dtype, ws, ws_bytes, stream);
    // float32 tensors (K = V = 64): the chunked float32 backward over the packed sequences
    const bool f32 = dtype == RWKV7_DTYPE_F32 && K == 64 && V == 64;
    int rc = check_seq(r, w, k, v, a, b, h0, h0_batch_stride, dr, nullptr, 1, T_total, H, K, V, dtype);
    if (rc != RWKV7_OK) return rc;
    rc = check_varlen(cu_seqlens, n_seq, T_total, H);
    if (rc != RWKV7_OK) return rc;
    if (!dw || !dk || !dv || !da || !db) return RWKV7_ERR_NULL_POINTER;
    if (!aligned16(d_o) || !aligned16(d_ht) || !aligned16(dw) || !aligned16(dk) || !aligned16(dv) ||
        !aligned16(da) || !aligned16(db) || !aligned16(dh0))
        return RWKV7_ERR_ALIGNMENT;
    const size_t need = f32 ? rwkv7::bwd_chunk_f32_workspace_bytes(n_seq, T_total, H, true)
                            : rwkv7::bwd_chunk_workspace_bytes(n_seq, T_total, H, true);
    if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return RWKV7_ERR_WORKSPACE;
    rwkv7::BwdArgs p;
    p.r = r; p.w = w; p.k = k; p.v = v; p.a = a; p.b = b;
    p.h0 = h0; p.h0_batch_stride = h0 ? h0_batch_stride : 0;
    p.dO = d_o; p.dht = d_ht;
    p.dr = dr; p.dw = dw; p.dk = dk; p.dv = dv; p.da = da; p.db = db; p.dh0 = dh0;
    p.B = n_seq; p.T = T_total; p.H = H; p.dtype = dtype; p.cu = cu_seqlens;
    if (f32) return (int)rwkv7::launch_bwd_chunk_f32(p, ws, static_cast<hipStream_t>(stream));
    return (int)rwkv7::launch_bwd_chunk(p, ws, static_cast<hipStream_t>(stream));
}

size_t rwkv7_bwd_recurrent_varlen_workspace_bytes(int n_seq, int T_total, int H, int K) {
    if (n_seq < 1 || T_total < 1 || H < 1 || (K != 64 && K != 128)) return 0;
    return rwkv7::bwd_recurrent_workspace_bytes(n_seq, T_total, H, K, true);
}

int rwkv7_bwd_recurrent_varlen(const void* r, const void* w, const void* k, const void* v, const void* a, const void* b,
                               const int32_t* cu_seqlens, int n_seq, const float* h0, int64_t h0_batch_stride,
                               const void* d_o, const float* d_ht,
                               void* dr, void* dw, void* dk, void* dv, void* da, void* db, float* dh0,
                               int T_total, int H, int K, int V, int dtype, void* ws, size_t ws_bytes, void* stream)
{
    int rc = check_seq(r, w, k, v, a, b, h0, h0_batch_stride, dr, nullptr, 1, T_total, H, K, V, dtype, true, true);
    if (rc != RWKV7_OK) return rc;
    rc = check_varlen(cu_seqlens, n_seq, T_total, H);
    if (rc != RWKV7_OK) return rc;
    if (!dw || !dk || !dv || !da || !db) return RWKV7_ERR_NULL_POINTER;
    if (!aligned16(d_o) || !aligned16(d_ht) || !aligned16(dw) || !aligned16(dk) || !aligned16(dv) ||
        !aligned16(da) || !aligned16(db) || !aligned16(dh0))
        return RWKV7_ERR_ALIGNMENT;
    const size_t need = rwkv7::bwd_recurrent_workspace_bytes(n_seq, T_total, H, K, true);
    if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return RWKV7_ERR_WORKSPACE;
    rwkv7::BwdArgs p;
    p.r = r; p.w = w; p.k = k; p.v = v; p.a = a; p.b = b;
    p.h0 = h0; p.h0_batch_stride = h0 ? h0_batch_stride : 0;
    p.dO = d_o; p.dht = d_ht;
    p.dr = dr; p.dw = dw; p.dk = dk; p.dv = dv; p.da = da; p.db = db; p.dh0 = dh0;
    p.B = n_seq; p.T = T_total; p.H = H; p.dtype = dtype; p.cu = cu_seqlens;
    return (int)rwkv7::launch_bwd_recurrent(p, K, ws, static_cast<hipStream_t>(stream));
}

/* ---- RWKV6 ------------------------------------------------------------------------------------- */
namespace {
int pack_rwkv6(const void* r, const void* k, const void* v, const void* w, const void* u,
               const float* states, int n_state, const int32_t* state_map, void* y, float* ys,
               int B, int T, int H, int K, int V, int dtype, SeqArgs& p)
{
    // a and b do not exist for this operator: r stands in for them in the common checks
    int rc = check_seq(r, w, k, v, r, r, states, (int64_t)H * K * V, y, ys, B, T, H, K, V, dtype, true);
    if (rc != RWKV7_OK) return rc;
    if (!u) return RWKV7_ERR_NULL_POINTER;
    if (!aligned16(u) || (reinterpret_cast<uintptr_t>(state_map) & 3u) != 0) return RWKV7_ERR_ALIGNMENT;
    if (states != nullptr) {
        if (n_state < 1) return RWKV7_ERR_BAD_SHAPE;
        if (state_map == nullptr && n_state != 1 && n_state != B) return RWKV7_ERR_BAD_SHAPE;
    } else if (state_map != nullptr) {
        return RWKV7_ERR_NULL_POINTER;
    }
    p = pack(r, w, k, v, nullptr, nullptr, states,
             (states && !state_map && n_state == 1 && B != 1) ? 0 : (int64_t)H * K * V, y, ys, B, T, H, dtype, K);
    p.u6 = u;
    if (states && state_map) { p.h0_map = state_map; p.n_state = n_state; }
    return RWKV7_OK;
}
}  // namespace

size_t rwkv6_fwd_workspace_bytes(int B, int T, int H, int dtype) {
    return rwkv7_fwd_workspace_bytes(B, T, H, dtype);        // the same kernels in their RWKV6 mode
}

int rwkv6_fwd(const void* r, const void* k, const void* v, const void* w, const void* u,
              const float* states, int n_state, const int32_t* state_map, void* y, float* ys,
              int B, int T, int H, int K, int V, int dtype, void* ws, size_t ws_bytes, void* stream)
{
    SeqArgs p;
    int rc = pack_rwkv6(r, k, v, w, u, states, n_state, state_map, y, ys, B, T, H, K, V, dtype, p);
    if (rc != RWKV7_OK) return rc;
    if (T == 1) return (int)rwkv7::launch_decode(p, static_cast<hipStream_t>(stream));
    if (dtype == RWKV7_DTYPE_F32 || T <= RECURRENT_MAX_T || K == 128)
        return (int)rwkv7::launch_rwkv6_recurrent(p, static_cast<hipStream_t>(stream));
    const size_t need = rwkv6_fwd_workspace_bytes(B, T, H, dtype);
    if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return RWKV7_ERR_WORKSPACE;
    if (use_fused_forward(B, H)) return (int)rwkv7::launch_fwd_fused(p, ws, static_cast<hipStream_t>(stream));
    return (int)rwkv7::launch_fwd_chunk(p, ws, static_cast<hipStream_t>(stream));
}

int rwkv6_fwd_recurrent(const void* r, const void* k, const void* v, const void* w, const void* u,
                        const float* states, int n_state, const int32_t* state_map, void* y, float* ys,
                        int B, int T, int H, int K, int V, int dtype, void* stream)
{
    SeqArgs p;
    int rc = pack_rwkv6(r, k, v, w, u, states, n_state, state_map, y, ys, B, T, H, K, V, dtype, p);
    if (rc != RWKV7_OK) return rc;
    return (int)rwkv7::launch_rwkv6_recurrent(p, static_cast<hipStream_t>(stream));
}

size_t rwkv6_bwd_workspace_bytes_head(int B, int T, int H, int K, int dtype) {
    if ((dtype != RWKV7_DTYPE_BF16 && dtype != RWKV7_DTYPE_F32) || B < 1 || T < 1 || H < 1 || (K != 64 && K != 128))
        return 0;
    return rwkv7::rwkv6_bwd_workspace_bytes(B, T, H, K, dtype);
}

size_t rwkv6_bwd_workspace_bytes(int B, int T, int H, int dtype) {
    return rwkv6_bwd_workspace_bytes_head(B, T, H, 64, dtype);
}

int rwkv6_bwd(const void* r, const void* k, const void* v, const void* w, const void* u, const void* d_y,
              void* dr, void* dk, void* dv, void* dw, float* du,
              int B, int T, int H, int K, int V, int dtype, void* ws, size_t ws_bytes, void* stream)
{
    if (dtype == RWKV7_DTYPE_F16) return RWKV7_ERR_UNSUPPORTED;
    int rc = check_seq(r, w, k, v, r, r, nullptr, 0, dr, nullptr, B, T, H, K, V, dtype, true);
    if (rc != RWKV7_OK) return rc;
    // the state path runs as 2B - 1 packed sequences over B*T - 1 tokens
    if ((((int64_t)B * T) >> 6) + 2 * (int64_t)B > ((int64_t)1 << 30) / H) return RWKV7_ERR_BAD_SHAPE;
    if (!u || !d_y || !dk || !dv || !dw || !du) return RWKV7_ERR_NULL_POINTER;
    if (!aligned16(u) || !aligned16(d_y) || !aligned16(dk) || !aligned16(dv) || !aligned16(dw) || !aligned16(du))
        return RWKV7_ERR_ALIGNMENT;
    const size_t need = rwkv7::rwkv6_bwd_workspace_bytes(B, T, H, K, dtype);
    if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0) return RWKV7_ERR_WORKSPACE;
    return (int)rwkv7::launch_rwkv6_bwd(r, k, v, w, u, d_y, dr, dk, dv, dw, du, B, T, H, K, dtype, ws,
                                        static_cast<hipStream_t>(stream));
}

}  // extern "C"
