// Float32 recurrent forward of the RWKV7 generalized delta rule for gfx950.
//
// The reference's native loop (/root/reference/rwkv_ops/rwkv7_kernel/native_keras_op.py:80-88)
// one token at a time, all arithmetic in float32 whatever the input type.  The state stays in
// registers for the whole sequence, laid out like the decode kernel's: the value columns are independent,
// so one wave64 owns CPW of them (N / CPW waves per (batch, head), one workgroup); with VQ = CPW / 4, lane =
// (ks = lane / VQ, vq = lane % VQ) holds N / (64 / VQ) rows of columns CPW*wave + 4*vq .. +3; the two
// contractions over K are in-register FMAs plus a cross-lane reduction over the 64 / VQ row groups (DPP
// rotations and lane swaps, no LDS).  K = 64 runs with CPW = 16 (four waves per head, about 130 instructions
// per wave and token: 0.46 us per token against 0.59 with CPW = 32), K = 128 with CPW = 32 (eight waves per
// head were no faster for one sequence and slower for many), or, when there are fewer (batch, head) pairs than
// CUs, as two workgroups per pair with CPW = 16 and half of the value columns each.  The per-token vectors
// come in blocks of 16 tokens: the workgroup requests a block with 16-byte loads while it computes the
// block before it, then converts it to float32 into LDS (w already as the decay exp(-exp(w))), from
// where every lane reads the entries of its rows.  What is left per token is the chain state -> a^T h ->
// state: the accurate path for float32 inputs, the only path for K = V = 128 with T > 1, and the
// on-device cross-check of the chunked kernels, not the throughput path.
#include "rwkv7_common.h"
#include "rwkv7_kernels.h"
#include "../../include/rwkv7_mi355x.h"

namespace rwkv7 {

namespace {
// Sums over the lanes that share lane % VQ (VQ = 4: sixteen lanes, VQ = 8: eight).
// the part of that sum inside a 16-lane row
template <int VQ>
__device__ __forceinline__ float reduce_in_row(float x) {
    if constexpr (VQ == 4)
        x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x124, 0xf, 0xf, true));   // row_ror:4
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x128, 0xf, 0xf, true));       // row_ror:8
    return x;
}
// the four components of v summed over the row groups, to all lanes (two registers per lane swap: rwkv7_common.h)
template <int VQ>
__device__ __forceinline__ void reduce_row_groups4(float4_t& v) {
    float a = reduce_in_row<VQ>(v.x), b = reduce_in_row<VQ>(v.y), c = reduce_in_row<VQ>(v.z), d = reduce_in_row<VQ>(v.w);
    sum4_over_rows(a, b, c, d);
    v = float4_t{a, b, c, d};
}
// ... component r to the 16-lane row r of the wave only
template <int VQ>
__device__ __forceinline__ float reduce_row_groups4_scattered(const float4_t& v) {
    return sum4_over_rows_scattered(reduce_in_row<VQ>(v.x), reduce_in_row<VQ>(v.y), reduce_in_row<VQ>(v.z), reduce_in_row<VQ>(v.w));
}
constexpr int REC_TB = 16;                       // tokens per staged block
}  // namespace

// V6 = true is the RWKV6 operator (/root/reference/rwkv_ops/rwkv6_kernel/ops_rwkv_kernel.py:65-73):
// o = r^T (diag(u) k v^T + h),  h <- k v^T + diag(d) h, with u [H][N] passed in b's place and a unused.
// VS = 2: the value columns of a head over two workgroups (blockIdx.x = (batch, head) * 2 + half), for calls with
// fewer heads than CUs; the columns being independent, the halves share nothing.
template <typename T, int N, bool V6 = false, int VS = 1, int CPW = (N == 64 ? 16 : 32) / VS>
__global__ __launch_bounds__(64 * (N / VS / CPW))
void fwd_recurrent_kernel(const T* __restrict__ r, const T* __restrict__ w, const T* __restrict__ k,
                          const T* __restrict__ v, const T* __restrict__ a, const T* __restrict__ b,
                          const float* __restrict__ h0, int64_t h0_batch_stride,
                          const int* __restrict__ h0_map, int n_state,
                          T* __restrict__ o, float* __restrict__ ht, SeqLayout L,
                          float* __restrict__ seg_states = nullptr, int seg = 0)
{
    // seg_states: the state BEFORE token t is stored for every t that is a multiple of `seg` (a multiple of REC_TB):
    // what the recurrent backward restarts from; o may then be NULL.  Dense batches: [workgroup][t / seg][N][N].
    // Packed sequences: sequence b owns the slots from (first row / seg) + b on (at most len / seg + 1 of them, never
    // the next sequence's), record (slot + t / seg) H + h; (T_total / seg + n_seq) H records in all.
    constexpr int VQ = CPW / 4;                  // lanes across a wave's columns, four columns each
    constexpr int ROWS = N / (64 / VQ);          // state rows per lane
    constexpr int NT = 64 * (N / VS / CPW);      // threads
    constexpr int PER16 = 16 / (int)sizeof(T);   // elements per 16-byte load
    constexpr int PIECES = 6 * REC_TB * N / PER16 / NT;    // 16-byte loads per thread and block
    __shared__ __attribute__((aligned(16))) float stage[6][REC_TB][N];   // a, d, b, k, r, v
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int bh = blockIdx.x / VS;
    const int col0 = (N / VS) * (blockIdx.x % VS) + CPW * (tid >> 6);    // the wave's first value column
    const int H = L.H;
    const int bi = bh / H, hi = bh % H;
    const SeqSpan sp = seq_span(L, bi);
    const int T_len = sp.len;
    const int ks = lane / VQ, vq = lane % VQ;
    const int tile = (ROWS * ks) * N + col0 + 4 * vq;

    float4_t s[ROWS];
    if (h0 != nullptr) {
        const float* src = h0 + state_row(h0_map, n_state, bi) * h0_batch_stride + (int64_t)hi * (N * N) + tile;
#pragma unroll
        for (int i = 0; i < ROWS; ++i) s[i] = *reinterpret_cast<const float4_t*>(src + i * N);
    } else {
#pragma unroll
        for (int i = 0; i < ROWS; ++i) s[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    }

    const T* const tensors[6] = {a, w, b, k, r, v};
    auto skipped = [](int q) { return V6 && (q == 0 || q == 2); };    // RWKV6 has no per-token a and b
    float uv[ROWS];
    if constexpr (V6) load_n<T, ROWS>(b + (int64_t)hi * N + ROWS * ks, uv);
    const int64_t step = (int64_t)H * N;
    const int64_t base = (sp.tok0 * H + hi) * N;
    // piece p of a thread: 16 bytes of tensor q, token tt of the block, elements e0 .. e0 + PER16 - 1
    u32x4_t raw[PIECES];
    auto request = [&](int t0) {
#pragma unroll
        for (int p = 0; p < PIECES; ++p) {
            const int c = p * NT + tid;
            const int q = c / (REC_TB * N / PER16), rem = c % (REC_TB * N / PER16);
            const int tt = rem / (N / PER16), e0 = (rem % (N / PER16)) * PER16;
            if (!skipped(q) && t0 + tt < T_len)
                raw[p] = *reinterpret_cast<const u32x4_t*>(tensors[q] + base + (t0 + tt) * step + e0);
        }
    };
    auto deposit = [&]() {
#pragma unroll
        for (int p = 0; p < PIECES; ++p) {
            const int c = p * NT + tid;
            const int q = c / (REC_TB * N / PER16), rem = c % (REC_TB * N / PER16);
            const int tt = rem / (N / PER16), e0 = (rem % (N / PER16)) * PER16;
            if (skipped(q)) continue;
            float x[PER16];
            if constexpr (sizeof(T) == 4) {
                x[0] = __uint_as_float(raw[p].x); x[1] = __uint_as_float(raw[p].y);
                x[2] = __uint_as_float(raw[p].z); x[3] = __uint_as_float(raw[p].w);
            } else {
                const uint32_t u[4] = {raw[p].x, raw[p].y, raw[p].z, raw[p].w};
#pragma unroll
                for (int m = 0; m < 4; ++m) {
                    if constexpr (sizeof(T) == 2 && !__is_same(T, bf16_t)) {          // float16
                        typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
                        const f16x2_t h2 = __builtin_bit_cast(f16x2_t, u[m]);
                        x[2 * m] = (float)h2[0];
                        x[2 * m + 1] = (float)h2[1];
                    } else {
                        x[2 * m] = bf16_bits_to_f32(u[m] & 0xffffu);
                        x[2 * m + 1] = __uint_as_float(u[m] & 0xffff0000u);
                    }
                }
            }
            if (q == 1) {
#pragma unroll
                for (int m = 0; m < PER16; ++m) x[m] = decay_from_w(x[m]);
            }
#pragma unroll
            for (int m = 0; m < PER16; m += 4)
                *reinterpret_cast<float4_t*>(&stage[q][tt][e0 + m]) = float4_t{x[m], x[m + 1], x[m + 2], x[m + 3]};
        }
    };

    request(0);
    for (int t0 = 0; t0 < T_len; t0 += REC_TB) {
        __syncthreads();                         // the block before this one has been consumed
        deposit();
        __syncthreads();
        request(t0 + REC_TB);
        if (seg_states != nullptr && t0 % seg == 0) {
            const int nseg = (T_len + seg - 1) / seg;
            const int64_t rec = L.cu != nullptr ? (sp.tok0 / seg + bi + t0 / seg) * H + hi
                                                : (int64_t)bh * nseg + t0 / seg;
            float* dst = seg_states + rec * (N * N) + tile;
#pragma unroll
            for (int i = 0; i < ROWS; ++i) *reinterpret_cast<float4_t*>(dst + i * N) = s[i];
        }
        const int nt = T_len - t0 < REC_TB ? T_len - t0 : REC_TB;
#pragma unroll 4
        for (int tt = 0; tt < nt; ++tt) {
            float av[ROWS], d[ROWS], bv[ROWS], kv[ROWS], rv[ROWS];
#pragma unroll
            for (int i = 0; i < ROWS; i += 4) {
                const float4_t d4 = *reinterpret_cast<const float4_t*>(&stage[1][tt][ROWS * ks + i]);
                const float4_t a4 = V6 ? d4 : *reinterpret_cast<const float4_t*>(&stage[0][tt][ROWS * ks + i]);
                const float4_t b4 = V6 ? d4 : *reinterpret_cast<const float4_t*>(&stage[2][tt][ROWS * ks + i]);
                const float4_t k4 = *reinterpret_cast<const float4_t*>(&stage[3][tt][ROWS * ks + i]);
                const float4_t r4 = *reinterpret_cast<const float4_t*>(&stage[4][tt][ROWS * ks + i]);
#pragma unroll
                for (int m = 0; m < 4; ++m) { av[i + m] = a4[m]; d[i + m] = d4[m]; bv[i + m] = b4[m]; kv[i + m] = k4[m]; rv[i + m] = r4[m]; }
            }
            const float4_t v4 = *reinterpret_cast<const float4_t*>(&stage[5][tt][col0 + 4 * vq]);
            float4_t sa = {0.f, 0.f, 0.f, 0.f};
            if constexpr (!V6) {
#pragma unroll
                for (int i = 0; i < ROWS; ++i) sa += av[i] * s[i];
                reduce_row_groups4<VQ>(sa);
            }
            if (!V6 && o == nullptr) {                  // the states only
#pragma unroll
                for (int i = 0; i < ROWS; ++i) s[i] = d[i] * s[i] + bv[i] * sa + kv[i] * v4;
                continue;
            }
            float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < ROWS; ++i) {
                if constexpr (V6) {
                    const float4_t kv4 = kv[i] * v4;
                    acc += rv[i] * (uv[i] * kv4 + s[i]);        // reads the state before the step
                    s[i] = d[i] * s[i] + kv4;
                } else {
                    s[i] = d[i] * s[i] + bv[i] * sa + kv[i] * v4;
                    acc += rv[i] * s[i];
                }
            }
            const float o1 = reduce_row_groups4_scattered<VQ>(acc);    // row r of the wave: column col0 + 4 vq + r
            if ((lane & 15) < VQ && o != nullptr)
                Io<T>::store1(o + base + (t0 + tt) * step + col0 + 4 * vq + (lane >> 4), o1);
        }
    }
    if (ht != nullptr) {
        float* dst = ht + (int64_t)bh * (N * N) + tile;
#pragma unroll
        for (int i = 0; i < ROWS; ++i) *reinterpret_cast<float4_t*>(dst + i * N) = s[i];
    }
}

// head size 128 and fewer (batch, head) pairs than CUs: two workgroups per pair
constexpr int VSPLIT_MAX_BH = 192;

template <typename T, int N>
static hipError_t launch_t(const SeqArgs& p, hipStream_t stream, float* states = nullptr, int seg = 0) {
    const int n_bh = p.B * p.H;
    T* o = states != nullptr ? nullptr : (T*)p.o;
    float* ht = states != nullptr ? nullptr : p.ht;
    const int* map = states != nullptr ? nullptr : p.h0_map;
    if (N == 128 && n_bh <= VSPLIT_MAX_BH)
        fwd_recurrent_kernel<T, N, false, N == 128 ? 2 : 1><<<dim3((unsigned)(2 * n_bh)), dim3(256), 0, stream>>>(
            (const T*)p.r, (const T*)p.w, (const T*)p.k, (const T*)p.v, (const T*)p.a, (const T*)p.b,
            p.h0, p.h0_batch_stride, map, p.n_state, o, ht, seq_layout(p, nullptr), states, seg);
    else
        fwd_recurrent_kernel<T, N><<<dim3((unsigned)n_bh), dim3(256), 0, stream>>>(
            (const T*)p.r, (const T*)p.w, (const T*)p.k, (const T*)p.v, (const T*)p.a, (const T*)p.b,
            p.h0, p.h0_batch_stride, map, p.n_state, o, ht, seq_layout(p, nullptr), states, seg);
    return hipGetLastError();
}

template <typename T, int N>
static hipError_t launch_states_t(const SeqArgs& p, float* states, int seg, hipStream_t stream) {
    return launch_t<T, N>(p, stream, states, seg);
}

// the forward without outputs, storing the state at the start of every segment of `seg` tokens (dense batches, or
// packed sequences, p.cu: see the kernel for where the records go)
hipError_t launch_fwd_recurrent_states(const SeqArgs& p, float* states, int seg, hipStream_t stream) {
    if (p.N == 128)
        return p.dtype == RWKV7_DTYPE_BF16  ? launch_states_t<bf16_t, 128>(p, states, seg, stream)
               : p.dtype == RWKV7_DTYPE_F16 ? launch_states_t<f16_t, 128>(p, states, seg, stream)
                                            : launch_states_t<float, 128>(p, states, seg, stream);
    return p.dtype == RWKV7_DTYPE_BF16  ? launch_states_t<bf16_t, 64>(p, states, seg, stream)
           : p.dtype == RWKV7_DTYPE_F16 ? launch_states_t<f16_t, 64>(p, states, seg, stream)
                                        : launch_states_t<float, 64>(p, states, seg, stream);
}

template <typename T, int N>
static hipError_t launch6_t(const SeqArgs& p, hipStream_t stream) {
    fwd_recurrent_kernel<T, N, true><<<dim3((unsigned)(p.B * p.H)), dim3(256), 0, stream>>>(
        (const T*)p.r, (const T*)p.w, (const T*)p.k, (const T*)p.v, nullptr, (const T*)p.u6,
        p.h0, p.h0_batch_stride, p.h0_map, p.n_state, (T*)p.o, p.ht, seq_layout(p, nullptr));
    return hipGetLastError();
}

hipError_t launch_rwkv6_recurrent(const SeqArgs& p, hipStream_t stream) {
    if (p.N == 128)
        return p.dtype == RWKV7_DTYPE_BF16 ? launch6_t<bf16_t, 128>(p, stream) : launch6_t<float, 128>(p, stream);
    return p.dtype == RWKV7_DTYPE_BF16 ? launch6_t<bf16_t, HEAD>(p, stream) : launch6_t<float, HEAD>(p, stream);
}

hipError_t launch_fwd_recurrent(const SeqArgs& p, hipStream_t stream) {
    if (p.cu != nullptr) {             // rows of o behind the last sequence
        hipError_t e = launch_chunk_items(seq_layout(p, nullptr), nullptr, nullptr, 0, nullptr, tail_of_output(p), stream);
        if (e != hipSuccess) return e;
    }
    if (p.N == 128)
        return p.dtype == RWKV7_DTYPE_BF16  ? launch_t<bf16_t, 128>(p, stream)
               : p.dtype == RWKV7_DTYPE_F16 ? launch_t<f16_t, 128>(p, stream) : launch_t<float, 128>(p, stream);
    return p.dtype == RWKV7_DTYPE_BF16  ? launch_t<bf16_t, 64>(p, stream)
           : p.dtype == RWKV7_DTYPE_F16 ? launch_t<f16_t, 64>(p, stream) : launch_t<float, 64>(p, stream);
}

}  // namespace rwkv7
