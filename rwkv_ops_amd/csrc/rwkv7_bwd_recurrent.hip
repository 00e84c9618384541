// Float32 recurrent backward of the RWKV7 generalized delta rule for gfx950: the gradients of the
// reference's native loop (/root/reference/rwkv_ops/rwkv7_kernel/native_keras_op.py:80-88, which the
// reference differentiates with the host framework's autograd) one token at a time, all arithmetic in
// float32 whatever the input type, for K = V = 64 and 128.  It is the accurate path (float32 callers,
// head size 128, float16), not the throughput path: that is the chunked bf16 backward.
//
// Forward step (per batch and head, state h[K][V]):
//     sa = a^T h,   h' = diag(d) h + b sa^T + k v^T,   o = r^T h',   d = exp(-exp(w))
// Reverse step, with H the adjoint of h' (everything later already added) and h the state BEFORE the step:
//     H  += r do^T
//     dr  = h' do = d (h do) + b (sa . do) + k (v . do)
//     dk  = H v,   dv = H^T k,   db = H sa,   dd = rowsum(H * h),   dsa = H^T b
//     da  = h dsa,   dw = dd * d * (-exp(w))
//     H  <- diag(d) H + a dsa^T                    (adjoint of h)
// The reverse walk needs h before every step.  Two launches:
//   1. the recurrent forward kernel (rwkv7_fwd_recurrent.hip) run once more, storing the state at the start of
//      every segment of SEG tokens;
//   2. bwd_recurrent_kernel, one workgroup per (batch, head), segments last to first: it re-runs the segment
//      forward from its stored state, writing the state before each token to a per-workgroup scratch area (and
//      sa to LDS), then walks the segment backwards.
// Layout: that of the forward kernel -- a wave owns CPW value columns, lane (ks, vq) holds ROWS rows of four of
// them, for h and H alike.  Sums over K (sa, dv, dsa: the ones on the chain) are in-register plus the forward
// kernel's cross-lane reduction inside the wave; sums over V (dr, dk, db, dd, da) cross the waves, but nothing
// later depends on them, so each wave leaves its partial sums in LDS and the workgroup adds them up and writes
// the five output rows once per block of RB_TB tokens.
#include "rwkv7_common.h"
#include "rwkv7_kernels.h"
#include "../../include/rwkv7_mi355x.h"

namespace rwkv7 {

namespace {

constexpr int RB_TB = 8;                         // tokens per staged block

template <int VQ>
__device__ __forceinline__ float reduce_rows(float x) {      // sum over the lanes that share lane % VQ
    if constexpr (VQ == 4)
        x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x124, 0xf, 0xf, true));   // row_ror:4
    return sum_lane_groups_of_8(x);
}

// sum over the VQ adjacent lanes that share lane / VQ (the columns of one row group), delivered to lane % VQ == 0
template <int VQ>
__device__ __forceinline__ float reduce_cols(float x) {
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x101, 0xf, 0xf, true));       // row_shl:1
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x102, 0xf, 0xf, true));       // row_shl:2
    if constexpr (VQ == 8)
        x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x104, 0xf, 0xf, true));   // row_shl:4
    return x;
}

__device__ __forceinline__ float dot4(float4_t a, float4_t b) { return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w; }

template <int N, int VS = 1> struct RecShape {
    static constexpr int CPW = (N == 64 ? 16 : 32) / VS;     // value columns per wave (four waves cover N / VS columns)
    static constexpr int SEG = N == 64 ? 64 : 32;            // tokens per segment
};
// Head size 128 with few (batch, head) pairs: the value columns of a head go to VS = 2 workgroups (the walk is bound by
// the vector throughput of a CU, and half of the CUs would have no head); each leaves its partial sums of the five
// [token][key] gradients in the workspace and a small kernel adds them.
constexpr int VSPLIT_MAX_BH = 192;
bool splits_values(int B, int H, int N, bool varlen) { return N == 128 && !varlen && (int64_t)B * H <= VSPLIT_MAX_BH; }

}  // namespace

int bwd_recurrent_segment(int N) { return N == 64 ? RecShape<64>::SEG : RecShape<128>::SEG; }

namespace {
// packed sequences: (T_total / seg + n_seq) H records; scratch areas for at most WALK_MAX_GRID workgroups
size_t rec_records(int B, int T, int H, int seg, bool varlen) {
    return varlen ? ((size_t)(T / seg) + B) * H : (size_t)B * H * ((T + seg - 1) / seg);
}
size_t rec_areas(int B, int H, bool varlen) {
    const size_t bh = (size_t)B * H;
    return varlen && bh > (size_t)WALK_MAX_GRID ? (size_t)WALK_MAX_GRID : bh;
}
}  // namespace

size_t bwd_recurrent_workspace_bytes(int B, int T, int H, int N, bool varlen) {
    const int seg = bwd_recurrent_segment(N);
    const size_t state = (size_t)N * N * 4;
    const bool split = splits_values(B, H, N, varlen);
    // stored segment states, then each workgroup's scratch, then (value columns split over two workgroups) the two
    // parts' sums of the five [token][key] gradients
    return (rec_records(B, T, H, seg, varlen) + rec_areas(B, H, varlen) * (split ? 2 : 1) * seg) * state +
           (split ? (size_t)2 * 5 * B * T * H * N * 4 : 0);
}

template <typename T, int N, int VS = 1>
__global__ __launch_bounds__(256)
void bwd_recurrent_kernel(const T* __restrict__ r, const T* __restrict__ w, const T* __restrict__ k,
                          const T* __restrict__ v, const T* __restrict__ a, const T* __restrict__ b,
                          const T* __restrict__ d_o, const float* __restrict__ d_ht,
                          const float* __restrict__ ckpt, float* __restrict__ scratch,
                          T* __restrict__ dr, T* __restrict__ dw, T* __restrict__ dk, T* __restrict__ dv,
                          T* __restrict__ da, T* __restrict__ db, float* __restrict__ dh0, int T_rows, int H,
                          int ckpt_per_head, int ckpt_step, const int* __restrict__ run_if_any, int n_flags,
                          const int* __restrict__ cu, int n_bh, int cu_shift, float* __restrict__ pbuf)
{
    // VS > 1 (dense batches): workgroup item = (batch, head) * VS + part owns the value columns (N / VS) * part .. of
    // its head and writes its sums over them of dr, dk, db, dw, da to pbuf [VS][5][B * T_rows][H][N] (float32).
    // ckpt: the state before token SEG * s is record ckpt_step * s of this head's ckpt_per_head records.
    // run_if_any (nullable): n_flags integers; the kernel runs only when one of them is not zero.
    // cu (nullable): packed sequences -- cumulative lengths of the n_bh / H sequences in one row of T_rows tokens;
    // the checkpoints are then records of one per 2^cu_shift tokens laid out by slots (sequence b, segment s: record
    // ((first row >> cu_shift) + b + s (SEG >> cu_shift)) H + h): cu_shift 4 for the records of the chunked float32
    // backward, log2(SEG) for this backward's own forward pass.  The grid may be smaller than n_bh: a workgroup takes
    // every gridDim.x-th (sequence, head) and owns one scratch area.
    constexpr int CPW = RecShape<N, VS>::CPW, SEG = RecShape<N, VS>::SEG;
    constexpr int VQ = CPW / 4;                  // lanes across a wave's columns, four columns each
    constexpr int ROWS = N / (64 / VQ);          // state rows per lane
    constexpr int PARTS = N / VS / CPW;          // waves
    static_assert(PARTS == 4, "four waves per workgroup");
    // staged per-token vectors of one block, as float: a, d, b, k, v (both passes), r, do, dfac (reverse pass)
    enum { Q_A = 0, Q_D, Q_B, Q_K, Q_V, Q_R, Q_DO, Q_DF, Q_COUNT };
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    float (*stage)[RB_TB][N] = reinterpret_cast<float (*)[RB_TB][N]>(smem_raw);
    float (*sa_buf)[N] = reinterpret_cast<float (*)[N]>(smem_raw + sizeof(float) * Q_COUNT * RB_TB * N);
    // partial sums over a wave's columns: [output][token of the block][wave][row]
    float (*part)[RB_TB][PARTS][N] = reinterpret_cast<float (*)[RB_TB][PARTS][N]>(
        smem_raw + sizeof(float) * (Q_COUNT * RB_TB * N + SEG * N));
    enum { O_DR = 0, O_DK, O_DB, O_DD, O_DA, O_COUNT };

    const int tid = threadIdx.x;
    if (run_if_any != nullptr) {
        int mine = 0;
        for (int i = tid; i < n_flags; i += 256) mine |= run_if_any[i];
        if (__syncthreads_or(mine) == 0) return;
    }
    const int lane = tid & 63;
    const int wave = tid >> 6;                   // which CPW value columns
    const int ks = lane / VQ, vq = lane % VQ;
    const int row0 = ROWS * ks;                  // this lane's first state row
    const int64_t step = (int64_t)H * N;
    float* my_scr = scratch + (int64_t)blockIdx.x * SEG * (N * N);
  for (int item = blockIdx.x; item < n_bh * VS; item += gridDim.x) {
    const int bh = item / VS, vs = item % VS;
    const int col0 = (N / VS) * vs + CPW * wave + 4 * vq;    // this lane's four value columns
    const int tile = row0 * N + col0;
    const int hi = bh % H, bi = bh / H;
    int64_t tok0 = (int64_t)bi * T_rows;
    int T_len = T_rows;
    if (cu != nullptr) {
        int s0 = load_table(cu + bi), e0 = load_table(cu + bi + 1);
        s0 = s0 < 0 ? 0 : (s0 > T_rows ? T_rows : s0);
        e0 = e0 < s0 ? s0 : (e0 > T_rows ? T_rows : e0);
        tok0 = s0; T_len = e0 - s0;
    }
    const int64_t base = (tok0 * H + hi) * N;
    const int nseg = (T_len + SEG - 1) / SEG;
    const float* my_ckpt = cu != nullptr ? ckpt + (((tok0 >> cu_shift) + bi) * H + hi) * (int64_t)(N * N)
                                         : ckpt + (int64_t)bh * ckpt_per_head * (N * N);
    const int64_t ckpt_stride = cu != nullptr ? (int64_t)(SEG >> cu_shift) * H * (N * N) : (int64_t)ckpt_step * (N * N);

    // one block of per-token vectors -> LDS as float (w as the decay d, and as dfac = dd/dw = -exp(w) d)
    auto stage_block = [&](int t0, int nt, bool reverse_pass) {
        for (int idx = tid; idx < RB_TB * (N / 4); idx += 256) {
            const int tt = idx / (N / 4), e0 = (idx % (N / 4)) * 4;
            if (tt >= nt) continue;
            const int64_t off = base + (int64_t)(t0 + tt) * step + e0;
            float x[4];
            Io<T>::load4(a + off, x);
            *reinterpret_cast<float4_t*>(&stage[Q_A][tt][e0]) = float4_t{x[0], x[1], x[2], x[3]};
            Io<T>::load4(b + off, x);
            *reinterpret_cast<float4_t*>(&stage[Q_B][tt][e0]) = float4_t{x[0], x[1], x[2], x[3]};
            Io<T>::load4(k + off, x);
            *reinterpret_cast<float4_t*>(&stage[Q_K][tt][e0]) = float4_t{x[0], x[1], x[2], x[3]};
            Io<T>::load4(v + off, x);
            *reinterpret_cast<float4_t*>(&stage[Q_V][tt][e0]) = float4_t{x[0], x[1], x[2], x[3]};
            Io<T>::load4(w + off, x);
            float dd[4], df[4];
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                const float ew = __expf(x[m]);
                dd[m] = __expf(-ew);
                df[m] = -ew * dd[m];
            }
            *reinterpret_cast<float4_t*>(&stage[Q_D][tt][e0]) = float4_t{dd[0], dd[1], dd[2], dd[3]};
            if (reverse_pass) {
                *reinterpret_cast<float4_t*>(&stage[Q_DF][tt][e0]) = float4_t{df[0], df[1], df[2], df[3]};
                Io<T>::load4(r + off, x);
                *reinterpret_cast<float4_t*>(&stage[Q_R][tt][e0]) = float4_t{x[0], x[1], x[2], x[3]};
                if (d_o != nullptr) Io<T>::load4(d_o + off, x);
                else x[0] = x[1] = x[2] = x[3] = 0.f;
                *reinterpret_cast<float4_t*>(&stage[Q_DO][tt][e0]) = float4_t{x[0], x[1], x[2], x[3]};
            }
        }
    };
    auto rows_of = [&](int q, int tt, float (&x)[ROWS]) {
#pragma unroll
        for (int i = 0; i < ROWS; i += 4) {
            const float4_t t4 = *reinterpret_cast<const float4_t*>(&stage[q][tt][row0 + i]);
            x[i] = t4.x; x[i + 1] = t4.y; x[i + 2] = t4.z; x[i + 3] = t4.w;
        }
    };
    auto cols_of = [&](int q, int tt) { return *reinterpret_cast<const float4_t*>(&stage[q][tt][col0]); };

    // adjoint of the state after the last token
    float4_t Hd[ROWS];
    if (d_ht != nullptr) {
        const float* src = d_ht + (int64_t)bh * (N * N) + tile;
#pragma unroll
        for (int i = 0; i < ROWS; ++i) Hd[i] = *reinterpret_cast<const float4_t*>(src + i * N);
    } else {
#pragma unroll
        for (int i = 0; i < ROWS; ++i) Hd[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    }

    for (int seg = nseg - 1; seg >= 0; --seg) {
        const int s0 = seg * SEG;
        const int slen = T_len - s0 < SEG ? T_len - s0 : SEG;
        // ---- the segment forward once more: the state before each token -> scratch, sa -> LDS
        {
            float4_t s[ROWS];
            const float* src = my_ckpt + (int64_t)seg * ckpt_stride + tile;
#pragma unroll
            for (int i = 0; i < ROWS; ++i) s[i] = *reinterpret_cast<const float4_t*>(src + i * N);
            for (int t0 = 0; t0 < slen; t0 += RB_TB) {
                const int nt = slen - t0 < RB_TB ? slen - t0 : RB_TB;
                __syncthreads();                 // the block before this one has been consumed
                stage_block(s0 + t0, nt, false);
                __syncthreads();
                for (int tt = 0; tt < nt; ++tt) {
                    float av[ROWS], d[ROWS], bv[ROWS], kv[ROWS];
                    rows_of(Q_A, tt, av); rows_of(Q_D, tt, d); rows_of(Q_B, tt, bv); rows_of(Q_K, tt, kv);
                    const float4_t v4 = cols_of(Q_V, tt);
                    float* dst = my_scr + (int64_t)(t0 + tt) * (N * N) + tile;
                    float4_t sa = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int i = 0; i < ROWS; ++i) {
                        *reinterpret_cast<float4_t*>(dst + i * N) = s[i];
                        sa += av[i] * s[i];
                    }
                    sa.x = reduce_rows<VQ>(sa.x); sa.y = reduce_rows<VQ>(sa.y);
                    sa.z = reduce_rows<VQ>(sa.z); sa.w = reduce_rows<VQ>(sa.w);
                    if (ks == 0) *reinterpret_cast<float4_t*>(&sa_buf[t0 + tt][col0]) = sa;
#pragma unroll
                    for (int i = 0; i < ROWS; ++i) s[i] = d[i] * s[i] + bv[i] * sa + kv[i] * v4;
                }
            }
        }
        // ---- the segment backwards, block by block (the last, possibly short, block first)
        const int nblk = (slen + RB_TB - 1) / RB_TB;
        for (int blk = nblk - 1; blk >= 0; --blk) {
            const int t0 = blk * RB_TB;
            const int nt = slen - t0 < RB_TB ? slen - t0 : RB_TB;
            __syncthreads();                     // the block before: vectors consumed, partial sums written out;
                                                 // first block of the segment: the scratch stores above are done
            stage_block(s0 + t0, nt, true);
            __syncthreads();
            for (int tt = nt - 1; tt >= 0; --tt) {
                float4_t hp[ROWS];               // the state before this token
                const float* src = my_scr + (int64_t)(t0 + tt) * (N * N) + tile;
#pragma unroll
                for (int i = 0; i < ROWS; ++i) hp[i] = *reinterpret_cast<const float4_t*>(src + i * N);
                float av[ROWS], d[ROWS], bv[ROWS], kv[ROWS], rv[ROWS];
                rows_of(Q_A, tt, av); rows_of(Q_D, tt, d); rows_of(Q_B, tt, bv); rows_of(Q_K, tt, kv); rows_of(Q_R, tt, rv);
                const float4_t v4 = cols_of(Q_V, tt), do4 = cols_of(Q_DO, tt);
                const float4_t sa4 = *reinterpret_cast<const float4_t*>(&sa_buf[t0 + tt][col0]);
                const float sado = dot4(sa4, do4), vdo = dot4(v4, do4);
                float4_t dv4 = {0.f, 0.f, 0.f, 0.f}, dsa4 = {0.f, 0.f, 0.f, 0.f};
                float p_dr[ROWS], p_dk[ROWS], p_db[ROWS], p_dd[ROWS];
#pragma unroll
                for (int i = 0; i < ROWS; ++i) {
                    Hd[i] += rv[i] * do4;
                    p_dr[i] = d[i] * dot4(hp[i], do4) + bv[i] * sado + kv[i] * vdo;
                    p_dk[i] = dot4(Hd[i], v4);
                    p_db[i] = dot4(Hd[i], sa4);
                    p_dd[i] = dot4(Hd[i], hp[i]);
                    dv4 += kv[i] * Hd[i];
                    dsa4 += bv[i] * Hd[i];
                }
                dv4.x = reduce_rows<VQ>(dv4.x); dv4.y = reduce_rows<VQ>(dv4.y);
                dv4.z = reduce_rows<VQ>(dv4.z); dv4.w = reduce_rows<VQ>(dv4.w);
                dsa4.x = reduce_rows<VQ>(dsa4.x); dsa4.y = reduce_rows<VQ>(dsa4.y);
                dsa4.z = reduce_rows<VQ>(dsa4.z); dsa4.w = reduce_rows<VQ>(dsa4.w);
                if (ks == 0) {
                    const float o4[4] = {dv4.x, dv4.y, dv4.z, dv4.w};
                    Io<T>::store4(dv + base + (int64_t)(s0 + t0 + tt) * step + col0, o4);
                }
#pragma unroll
                for (int i = 0; i < ROWS; ++i) {
                    const float p_da = reduce_cols<VQ>(dot4(hp[i], dsa4));
                    const float s_dr = reduce_cols<VQ>(p_dr[i]), s_dk = reduce_cols<VQ>(p_dk[i]);
                    const float s_db = reduce_cols<VQ>(p_db[i]), s_dd = reduce_cols<VQ>(p_dd[i]);
                    if (vq == 0) {
                        part[O_DR][tt][wave][row0 + i] = s_dr;
                        part[O_DK][tt][wave][row0 + i] = s_dk;
                        part[O_DB][tt][wave][row0 + i] = s_db;
                        part[O_DD][tt][wave][row0 + i] = s_dd;
                        part[O_DA][tt][wave][row0 + i] = p_da;
                    }
                    Hd[i] = d[i] * Hd[i] + av[i] * dsa4;
                }
            }
            __syncthreads();
            // the five output rows of the block's tokens: sum over the four waves, four channels per thread
            for (int idx = tid; idx < nt * (N / 4); idx += 256) {
                const int tt = idx / (N / 4), e0 = (idx % (N / 4)) * 4;
                const int64_t off = base + (int64_t)(s0 + t0 + tt) * step + e0;
                T* const outs[O_COUNT] = {dr, dk, db, dw, da};
#pragma unroll
                for (int q = 0; q < O_COUNT; ++q) {
                    float4_t sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int p = 0; p < PARTS; ++p) sum += *reinterpret_cast<const float4_t*>(&part[q][tt][p][e0]);
                    if (q == O_DD) sum = sum * *reinterpret_cast<const float4_t*>(&stage[Q_DF][tt][e0]);
                    if constexpr (VS > 1) {
                        const int64_t all = (int64_t)(n_bh / H) * T_rows * step;       // elements of one tensor
                        *reinterpret_cast<float4_t*>(pbuf + ((int64_t)vs * O_COUNT + q) * all + off) = sum;
                    } else {
                        const float o4[4] = {sum.x, sum.y, sum.z, sum.w};
                        Io<T>::store4(outs[q] + off, o4);
                    }
                }
            }
        }
    }
    if (dh0 != nullptr) {
        float* dst = dh0 + (int64_t)bh * (N * N) + tile;
#pragma unroll
        for (int i = 0; i < ROWS; ++i) *reinterpret_cast<float4_t*>(dst + i * N) = Hd[i];
    }
    __syncthreads();                             // (the next (sequence, head) of this workgroup reuses the LDS areas)
  }
}

// out[q] = sum over the VS parts of pbuf [VS][5][elements], four elements per thread
template <typename T, int VS>
__global__ __launch_bounds__(256)
void bwd_recurrent_combine_kernel(const float* __restrict__ pbuf, T* __restrict__ dr, T* __restrict__ dk,
                                  T* __restrict__ db, T* __restrict__ dw, T* __restrict__ da, int64_t elements)
{
    const int64_t i4 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i4 >= elements) return;
    T* const outs[5] = {dr, dk, db, dw, da};      // the order of O_DR .. O_DA
#pragma unroll
    for (int q = 0; q < 5; ++q) {
        float4_t sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int p = 0; p < VS; ++p) sum += *reinterpret_cast<const float4_t*>(pbuf + ((int64_t)p * 5 + q) * elements + i4);
        const float o4[4] = {sum.x, sum.y, sum.z, sum.w};
        Io<T>::store4(outs[q] + i4, o4);
    }
}

namespace {
template <int N> constexpr size_t rec_lds_bytes() {
    return sizeof(float) * ((size_t)8 * RB_TB * N + (size_t)RecShape<N>::SEG * N + (size_t)5 * RB_TB * 4 * N);
}

template <typename T, int N, int VS = 1>
hipError_t launch_bwd_rec_t(const BwdArgs& p, const float* ckpt, float* scratch, hipStream_t stream,
                            int ckpt_per_head = 0, int ckpt_step = 1, const int* run_if_any = nullptr, int n_flags = 0,
                            int max_grid = 0, int cu_shift = 4, float* pbuf = nullptr) {
    if (ckpt_per_head == 0) ckpt_per_head = (p.T + RecShape<N>::SEG - 1) / RecShape<N>::SEG;
    const int n_bh = p.B * p.H;
    const int grid = max_grid > 0 && n_bh > max_grid ? max_grid : n_bh * VS;
    constexpr size_t lds = rec_lds_bytes<N>();
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(bwd_recurrent_kernel<T, N, VS>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    bwd_recurrent_kernel<T, N, VS><<<dim3((unsigned)grid), dim3(256), lds, stream>>>(
        (const T*)p.r, (const T*)p.w, (const T*)p.k, (const T*)p.v, (const T*)p.a, (const T*)p.b,
        (const T*)p.dO, p.dht, ckpt, scratch, (T*)p.dr, (T*)p.dw, (T*)p.dk, (T*)p.dv, (T*)p.da, (T*)p.db,
        p.dh0, p.T, p.H, ckpt_per_head, ckpt_step, run_if_any, n_flags, p.cu, n_bh, cu_shift, pbuf);
    e = hipGetLastError();
    if (e != hipSuccess || VS == 1) return e;
    const int64_t elements = (int64_t)p.B * p.T * p.H * N;
    bwd_recurrent_combine_kernel<T, VS><<<dim3((unsigned)((elements / 4 + 255) / 256)), dim3(256), 0, stream>>>(
        pbuf, (T*)p.dr, (T*)p.dk, (T*)p.db, (T*)p.dw, (T*)p.da, elements);
    return hipGetLastError();
}
}  // namespace

// the walk alone, for float32 tensors at K = V = 64, over states stored every 16 tokens (dense: record 4 s of a head
// = the state before token 64 s; packed (p.cu): the records of the chunked float32 backward); it runs only when one of
// the n_flags integers at run_if_any is not zero; at most WALK_MAX_GRID workgroups, each with a scratch area of 64 states
hipError_t launch_bwd_recurrent_walk_f32(const BwdArgs& p, const float* states16, float* scratch,
                                         const int* run_if_any, int n_flags, hipStream_t stream) {
    return launch_bwd_rec_t<float, 64>(p, states16, scratch, stream, (p.T + 15) / 16, 4, run_if_any, n_flags,
                                       p.cu != nullptr ? WALK_MAX_GRID : 0);
}

hipError_t launch_bwd_recurrent(const BwdArgs& p, int N, void* ws, hipStream_t stream) {
    const int seg = bwd_recurrent_segment(N);
    const bool varlen = p.cu != nullptr;
    float* ckpt = static_cast<float*>(ws);
    float* scratch = ckpt + rec_records(p.B, p.T, p.H, seg, varlen) * N * N;
    // launch 1: the forward once more, leaving the state at the start of every segment
    SeqArgs f{};
    f.r = p.r; f.w = p.w; f.k = p.k; f.v = p.v; f.a = p.a; f.b = p.b;
    f.h0 = p.h0; f.h0_batch_stride = p.h0 ? p.h0_batch_stride : 0;
    f.B = p.B; f.T = p.T; f.H = p.H; f.N = N; f.dtype = p.dtype; f.cu = p.cu;
    hipError_t e;
    if (varlen) {                      // rows of the gradients behind the last sequence
        TailFill tail;
        tail.p[0] = p.dr; tail.p[1] = p.dw; tail.p[2] = p.dk; tail.p[3] = p.dv; tail.p[4] = p.da; tail.p[5] = p.db;
        tail.n = 6; tail.row_bytes = (int64_t)p.H * N * (p.dtype == RWKV7_DTYPE_F32 ? 4 : 2);
        e = launch_chunk_items(seq_layout(f, nullptr), nullptr, nullptr, 0, nullptr, tail, stream);
        if (e != hipSuccess) return e;
    }
    // (dense float32 tensors at head size 64 beyond a dozen tokens: the chunked float32 forward, otherwise the recurrent one)
    e = (!varlen && N == 64 && p.dtype == RWKV7_DTYPE_F32 && p.T > 12) ? launch_fwd_chunk_f32_states(f, ckpt, seg, stream)
                                                                       : launch_fwd_recurrent_states(f, ckpt, seg, stream);
    if (e != hipSuccess) return e;
    // packed: the records lie by slots of one per segment, and at most WALK_MAX_GRID workgroups walk
    const int grid = varlen ? WALK_MAX_GRID : 0, shift = seg == 64 ? 6 : 5;
    if (splits_values(p.B, p.H, N, varlen)) {
        float* pbuf = scratch + (size_t)p.B * p.H * 2 * seg * N * N;
        return p.dtype == RWKV7_DTYPE_BF16  ? launch_bwd_rec_t<bf16_t, 128, 2>(p, ckpt, scratch, stream, 0, 1, nullptr, 0, 0, shift, pbuf)
               : p.dtype == RWKV7_DTYPE_F16 ? launch_bwd_rec_t<f16_t, 128, 2>(p, ckpt, scratch, stream, 0, 1, nullptr, 0, 0, shift, pbuf)
                                            : launch_bwd_rec_t<float, 128, 2>(p, ckpt, scratch, stream, 0, 1, nullptr, 0, 0, shift, pbuf);
    }
    if (N == 128)
        return p.dtype == RWKV7_DTYPE_BF16  ? launch_bwd_rec_t<bf16_t, 128>(p, ckpt, scratch, stream, 0, 1, nullptr, 0, grid, shift)
               : p.dtype == RWKV7_DTYPE_F16 ? launch_bwd_rec_t<f16_t, 128>(p, ckpt, scratch, stream, 0, 1, nullptr, 0, grid, shift)
                                            : launch_bwd_rec_t<float, 128>(p, ckpt, scratch, stream, 0, 1, nullptr, 0, grid, shift);
    return p.dtype == RWKV7_DTYPE_BF16  ? launch_bwd_rec_t<bf16_t, 64>(p, ckpt, scratch, stream, 0, 1, nullptr, 0, grid, shift)
           : p.dtype == RWKV7_DTYPE_F16 ? launch_bwd_rec_t<f16_t, 64>(p, ckpt, scratch, stream, 0, 1, nullptr, 0, grid, shift)
                                        : launch_bwd_rec_t<float, 64>(p, ckpt, scratch, stream, 0, 1, nullptr, 0, grid, shift);
}

}  // namespace rwkv7
