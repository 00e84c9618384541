// Backward of the RWKV6 operator (the call without a state, the one the reference differentiates:
// /root/reference/rwkv_ops/rwkv6_kernel/torch_rwkv_kernel.py:57-152, kernels in
// rwkv6_kernel/torch_kernel/wkv6_cuda.cu) on the RWKV7 backward kernels.
//
// With a = b = 0 the RWKV7 operator keeps RWKV6's state, s_t = diag(d_t) s_{t-1} + k_t v_t^T, and outputs
// o_t = r_t s_t, while RWKV6 outputs y_t = r_t s_{t-1} + (r_t . u * k_t) v_t.  Reading r and dy one token
// ahead, r'_t = r_{t+1}, turns one into the other: o'_t = y_{t+1} - bonus_{t+1}.  So the gradients of the
// state path are those of the RWKV7 operator on (r', w, k, v, 0, 0) with upstream gradient dy', its dr
// moved back by one token; the last token of a sequence takes no part (nothing reads the state after it).
// "One token ahead" is a pointer offset, and "without each sequence's last token" is a table of packed
// sequences: row b*T .. b*T+T-2 is sequence 2b, the single row b*T+T-1 is a dummy sequence 2b+1 whose
// results are discarded (the very last row is left out altogether, so no access leaves the tensors).
// An epilogue kernel adds the gradient of the bonus term and forms du.
#include "rwkv7_common.h"
#include "rwkv7_kernels.h"
#include "../../include/rwkv7_mi355x.h"

namespace rwkv7 {

namespace {

// cu[2b] = b*T, cu[2b+1] = b*T + T-1 (b < B), which ends at B*T - 1; and a zero-filled [B*T, H, N] tensor
// to stand for a and b
__global__ __launch_bounds__(256)
void rwkv6_bwd_prologue_kernel(int* __restrict__ cu, u32x4_t* __restrict__ zeros, int64_t n16, int B, int T)
{
    const int64_t i0 = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i0 < 2 * B) cu[i0] = (int)(i0 >> 1) * T + ((i0 & 1) ? T - 1 : 0);
    const u32x4_t z = {0u, 0u, 0u, 0u};
    for (int64_t i = i0; i < n16; i += (int64_t)gridDim.x * 256) zeros[i] = z;
}

// One workgroup per (batch, head, 64 tokens), lane = channel (N = 128: channels lane and lane + 64), wave v takes
// tokens v, v+4, ...:
//   s = <dy_t, v_t>, q = sum_c r u k;
//   dr_t = dr'_{t-1} + u k s,  dk_t = dk'_t + u r s,  dv_t = dv'_t + q dy_t,  dw_t = dw'_t,
// the primed terms being zero where the state path has none (t = 0 for dr, t = T-1 for the others; the
// buffers hold the dummy sequences' values or nothing there).  dk, dv, dw are corrected in place.
// du[h][c] = sum over batch and tokens of r k s: summed per workgroup, then one atomic per channel.
template <typename E, int N>
__global__ __launch_bounds__(256)
void rwkv6_bwd_epilogue_kernel(const E* __restrict__ r, const E* __restrict__ k,
                               const E* __restrict__ v, const E* __restrict__ u,
                               const E* __restrict__ dy, const E* __restrict__ dr_state,
                               E* __restrict__ dr, E* __restrict__ dk, E* __restrict__ dv,
                               E* __restrict__ dw, float* __restrict__ du, int T, int H, int state_path)
{
    constexpr int PER = N / 64;                  // channels per lane
    __shared__ float part[4][N];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int nblk = (T + 63) / 64;
    const int blk = blockIdx.x % nblk, hi = (blockIdx.x / nblk) % H, bi = blockIdx.x / (nblk * H);
    float uc[PER], du_acc[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) { uc[j] = (float)u[hi * N + lane + 64 * j]; du_acc[j] = 0.f; }
    for (int tt = wv; tt < 64; tt += 4) {
        const int t = blk * 64 + tt;
        if (t >= T) break;
        const int64_t row0 = (((int64_t)bi * T + t) * H + hi) * N + lane;
        float rc[PER], kc[PER], vc[PER], gc[PER];
        float s = 0.f, q = 0.f;
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int64_t row = row0 + 64 * j;
            rc[j] = (float)r[row]; kc[j] = (float)k[row]; vc[j] = (float)v[row]; gc[j] = (float)dy[row];
            s = fmaf(gc[j], vc[j], s);
            q = fmaf(rc[j] * uc[j], kc[j], q);
        }
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) { s += __shfl_xor(s, m, 64); q += __shfl_xor(q, m, 64); }
        const bool first = t == 0, last = t == T - 1;
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int64_t row = row0 + 64 * j;
            const float dr0 = (state_path && !first) ? (float)dr_state[row - (int64_t)H * N] : 0.f;
            const float dk0 = (state_path && !last) ? (float)dk[row] : 0.f;
            const float dv0 = (state_path && !last) ? (float)dv[row] : 0.f;
            dr[row] = (E)(dr0 + uc[j] * kc[j] * s);
            dk[row] = (E)(dk0 + uc[j] * rc[j] * s);
            dv[row] = (E)(dv0 + q * gc[j]);
            if (!state_path || last) dw[row] = (E)0.f;
            du_acc[j] = fmaf(rc[j] * kc[j], s, du_acc[j]);
        }
    }
#pragma unroll
    for (int j = 0; j < PER; ++j) part[wv][lane + 64 * j] = du_acc[j];
    __syncthreads();
    if (threadIdx.x < N)
        atomicAdd(du + hi * N + threadIdx.x,
                  part[0][threadIdx.x] + part[1][threadIdx.x] + part[2][threadIdx.x] + part[3][threadIdx.x]);
}

__global__ void rwkv6_zero_du_kernel(float* du, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) du[i] = 0.f;
}

size_t align256(size_t x) { return (x + 255) / 256 * 256; }

}  // namespace

// workspace: [cu table][zeros][dr of the state path][da, db dump][RWKV7 backward workspace]
// (N = 128: the state path is the float32 recurrent backward over the same table, as for RWKV7 at that head size)
size_t rwkv6_bwd_workspace_bytes(int B, int T, int H, int N, int dtype) {
    const bool f32 = dtype == RWKV7_DTYPE_F32;
    const size_t tensor = align256((size_t)B * T * H * N * (f32 ? 4 : 2));
    size_t n = align256((size_t)2 * B * 4) + 3 * tensor;
    if (T > 1) n += N == 128 ? bwd_recurrent_workspace_bytes(2 * B - 1, B * T - 1, H, 128, true)
                  : f32      ? bwd_chunk_f32_workspace_bytes(2 * B - 1, B * T - 1, H, true)
                             : bwd_chunk_workspace_bytes(2 * B - 1, B * T - 1, H, true);
    return n;
}

template <typename E, int N>
static void launch_epilogue(const void* r, const void* k, const void* v, const void* u, const void* dy,
                            const void* dr_state, void* dr, void* dk, void* dv, void* dw, float* du,
                            int B, int T, int H, hipStream_t stream)
{
    const int nblk = (T + 63) / 64;
    rwkv6_bwd_epilogue_kernel<E, N><<<dim3((unsigned)(B * H * nblk)), dim3(256), 0, stream>>>(
        (const E*)r, (const E*)k, (const E*)v, (const E*)u, (const E*)dy, (const E*)dr_state,
        (E*)dr, (E*)dk, (E*)dv, (E*)dw, du, T, H, T > 1 ? 1 : 0);
}

hipError_t launch_rwkv6_bwd(const void* r, const void* k, const void* v, const void* w, const void* u,
                            const void* dy, void* dr, void* dk, void* dv, void* dw, float* du,
                            int B, int T, int H, int N, int dtype, void* ws, hipStream_t stream)
{
    // float32 tensors: the same plan on the chunked float32 backward (every product on the float32 matrix cores),
    // so that float32 callers get float32 gradients as the reference's float32 kernel gives them
    // (/root/reference/rwkv_ops/rwkv6_kernel/torch_rwkv_kernel.py:137)
    const bool f32 = dtype == RWKV7_DTYPE_F32;
    const size_t tensor = align256((size_t)B * T * H * N * (f32 ? 4 : 2));
    unsigned char* base = static_cast<unsigned char*>(ws);
    int* cu = reinterpret_cast<int*>(base);
    unsigned char* zeros = base + align256((size_t)2 * B * 4);
    unsigned char* dr_state = zeros + tensor;
    unsigned char* dump = dr_state + tensor;
    void* bws = dump + tensor;
    rwkv6_zero_du_kernel<<<dim3((unsigned)((H * N + 255) / 256)), dim3(256), 0, stream>>>(du, H * N);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (T > 1) {
        const int64_t n16 = (int64_t)(tensor / 16);
        const int64_t want = (n16 + 255) / 256;
        rwkv6_bwd_prologue_kernel<<<dim3((unsigned)(want < 4096 ? (want < 1 ? 1 : want) : 4096)), dim3(256), 0, stream>>>(
            cu, reinterpret_cast<u32x4_t*>(zeros), n16, B, T);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
        const int64_t ahead = (int64_t)H * N * (f32 ? 4 : 2);             // one token, in bytes
        BwdArgs p;
        p.r = static_cast<const unsigned char*>(r) + ahead; p.w = w; p.k = k; p.v = v; p.a = zeros; p.b = zeros;
        p.h0 = nullptr; p.h0_batch_stride = 0;
        p.dO = static_cast<const unsigned char*>(dy) + ahead; p.dht = nullptr;
        p.dr = dr_state; p.dw = dw; p.dk = dk; p.dv = dv; p.da = dump; p.db = dump; p.dh0 = nullptr;
        p.B = 2 * B - 1; p.T = B * T - 1; p.H = H; p.dtype = dtype; p.cu = cu;
        e = N == 128 ? launch_bwd_recurrent(p, 128, bws, stream)
            : f32    ? launch_bwd_chunk_f32(p, bws, stream) : launch_bwd_chunk(p, bws, stream);
        if (e != hipSuccess) return e;
    }
    if (N == 128) {
        if (f32) launch_epilogue<float, 128>(r, k, v, u, dy, dr_state, dr, dk, dv, dw, du, B, T, H, stream);
        else launch_epilogue<bf16_t, 128>(r, k, v, u, dy, dr_state, dr, dk, dv, dw, du, B, T, H, stream);
    } else {
        if (f32) launch_epilogue<float, HEAD>(r, k, v, u, dy, dr_state, dr, dk, dv, dw, du, B, T, H, stream);
        else launch_epilogue<bf16_t, HEAD>(r, k, v, u, dy, dr_state, dr, dk, dv, dw, du, B, T, H, stream);
    }
    return hipGetLastError();
}

}  // namespace rwkv7
