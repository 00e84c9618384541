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
// The reverse walk needs h before every step.  Launches:
//   1. the recurrent forward kernel (rwkv7_fwd_recurrent.hip) run once more, storing the state at the start of
//      every segment of SEG tokens;
//   2. bwd_recurrent_kernel, one workgroup per (batch, head) (two at head size 128 when heads are few: VS below),
//      segments last to first: it re-runs the segment forward from its stored state, writing the state before
//      every KEEP-th token to a per-head scratch area (and sa of every token to LDS), then walks the segment
//      backwards in groups of KEEP tokens -- the kept state, requested a group ahead, and KEEP - 1 steps forward
//      from it;
//   3. with VS = 2, bwd_recurrent_combine_kernel adds the two halves' sums of dr, dk, db, dw, da.
// Layout: that of the forward kernel -- a wave owns CPW value columns, lane (ks, vq) holds ROWS rows of four of
// them, for h and H alike; W = 4 waves, or 8 at head size 128 (two waves per SIMD: one wave alone issues a vector
// instruction every 4 cycles, the SIMD takes one every 2).  Sums over K (sa, dv, dsa: the ones on the chain) are
// in-register plus the forward kernel's cross-lane reduction inside the wave; sums over V (dr, dk, db, dd, da)
// cross the waves, but nothing later depends on them, so each wave leaves its partial sums in LDS and the
// workgroup adds them up and writes the five output rows once per block of RB tokens.
#include <type_traits>
#include "rwkv7_common.h"
#include "rwkv7_kernels.h"
#include "../../include/rwkv7_mi355x.h"

namespace rwkv7 {

namespace {

// Sums over the lanes that share lane % VQ (the rows of the state that a wave holds): first inside a 16-lane row
template <int VQ>
__device__ __forceinline__ float reduce_rows_in_row(float x) {
    if constexpr (VQ == 2)
        x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x122, 0xf, 0xf, true));   // row_ror:2
    if constexpr (VQ <= 4)
        x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x124, 0xf, 0xf, true));   // row_ror:4
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x128, 0xf, 0xf, true));       // row_ror:8
    return x;
}
// then over the four rows, the four components of v at once (rwkv7_common.h), delivered to all lanes
template <int VQ>
__device__ __forceinline__ void reduce_rows4(float4_t& v) {
    float a = reduce_rows_in_row<VQ>(v.x), b = reduce_rows_in_row<VQ>(v.y);
    float c = reduce_rows_in_row<VQ>(v.z), d = reduce_rows_in_row<VQ>(v.w);
    sum4_over_rows(a, b, c, d);
    v = float4_t{a, b, c, d};
}
// ... delivered one component per 16-lane row: row r of the wave gets component r
template <int VQ>
__device__ __forceinline__ float reduce_rows4_scattered(const float4_t& v) {
    return sum4_over_rows_scattered(reduce_rows_in_row<VQ>(v.x), reduce_rows_in_row<VQ>(v.y),
                                    reduce_rows_in_row<VQ>(v.z), reduce_rows_in_row<VQ>(v.w));
}

// sum over the VQ adjacent lanes that share lane / VQ (the columns of one row group), delivered to lane % VQ == 0
template <int VQ>
__device__ __forceinline__ float reduce_cols(float x) {
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x101, 0xf, 0xf, true));       // row_shl:1
    if constexpr (VQ >= 4)
        x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x102, 0xf, 0xf, true));   // row_shl:2
    if constexpr (VQ == 8)
        x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x104, 0xf, 0xf, true));   // row_shl:4
    return x;
}

__device__ __forceinline__ float dot4(float4_t a, float4_t b) { return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w; }

template <int N, int VS = 1, int W = 4> struct RecShape {
    static constexpr int CPW = N / VS / W;                   // value columns per wave (W waves cover N / VS columns)
    static constexpr int SEG = N == 64 ? 64 : 32;            // tokens per segment
    static constexpr int RB = W * N > 512 ? 4 : 8;           // tokens per staged block (the partial sums fill 80 KiB of LDS)
    // The walk back keeps the state before every KEEP-th token of a segment and takes the others by steps forward
    // from it (three multiply-adds per element and no sum across lanes): a quarter of the scratch traffic, which
    // is what bounds the walk when there are more heads than CUs.
    static constexpr int KEEP = 4;
};
// Head size 128 with few (batch, head) pairs: the value columns of a head go to VS = 2 workgroups (the walk is bound by
// the vector throughput of a CU, and half of the CUs would have no head); each leaves its partial sums of the five
// [token][key] gradients in the workspace and a small kernel adds them.
constexpr int VSPLIT_MAX_BH = 192;
constexpr int W_SPLIT = 8, W_128 = 8, W_64 = 4;           // waves per workgroup
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
    return (rec_records(B, T, H, seg, varlen) + rec_areas(B, H, varlen) * seg) * state +
           (split ? (size_t)2 * 5 * B * T * H * N * 4 : 0);
}

template <typename T, int N, int VS = 1, int W = 4>
__global__ __launch_bounds__(64 * W)
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
    typedef RecShape<N, VS, W> Shape;
    constexpr int CPW = Shape::CPW, SEG = Shape::SEG, KEEP = Shape::KEEP, RB_TB = Shape::RB, NT = 64 * W;
    static_assert(RB_TB % KEEP == 0 && SEG % RB_TB == 0, "kept states at multiples of KEEP in every block");
    constexpr int VQ = CPW / 4;                  // lanes across a wave's columns, four columns each
    constexpr int ROWS = N / (64 / VQ);          // state rows per lane
    constexpr int PARTS = W;                     // waves
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
        for (int i = tid; i < n_flags; i += NT) mine |= run_if_any[i];
        if (__syncthreads_or(mine) == 0) return;
    }
    const int lane = tid & 63;
    const int wave = tid >> 6;                   // which CPW value columns
    const int ks = lane / VQ, vq = lane % VQ;
    const int row0 = ROWS * ks;                  // this lane's first state row
    const int64_t step = (int64_t)H * N;
    float* my_scr = scratch + (int64_t)(blockIdx.x / VS) * (SEG / KEEP) * (N * N);     // (the parts of a head share an area)
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

    // One block of per-token vectors -> LDS as float (w as the decay d, and as dfac = dd/dw = -exp(w) d), in two
    // halves: request() asks for the block while the block before it is being computed, deposit() converts what
    // has arrived.  reverse_pass adds r, do and dfac.
    typedef T tvec4 __attribute__((ext_vector_type(4)));
    constexpr int ITEMS = (RB_TB * (N / 4) + NT - 1) / NT;    // (token, four channels) items per thread
    tvec4 raw[ITEMS][7];                                      // a, b, k, v, w, r, do
    auto request = [&](int t0, int nt, bool reverse_pass) {
#pragma unroll
        for (int it = 0; it < ITEMS; ++it) {
            const int idx = it * NT + tid;
            const int tt = idx / (N / 4), e0 = (idx % (N / 4)) * 4;
            if (idx >= RB_TB * (N / 4) || tt >= nt) continue;
            const int64_t off = base + (int64_t)(t0 + tt) * step + e0;
            raw[it][0] = *reinterpret_cast<const tvec4*>(a + off);
            raw[it][1] = *reinterpret_cast<const tvec4*>(b + off);
            raw[it][2] = *reinterpret_cast<const tvec4*>(k + off);
            raw[it][3] = *reinterpret_cast<const tvec4*>(v + off);
            raw[it][4] = *reinterpret_cast<const tvec4*>(w + off);
            if (reverse_pass) {
                raw[it][5] = *reinterpret_cast<const tvec4*>(r + off);
                if (d_o != nullptr) raw[it][6] = *reinterpret_cast<const tvec4*>(d_o + off);
            }
        }
    };
    auto deposit = [&](int nt, bool reverse_pass) {
        auto as_float = [](const tvec4& x) { return float4_t{(float)x[0], (float)x[1], (float)x[2], (float)x[3]}; };
#pragma unroll
        for (int it = 0; it < ITEMS; ++it) {
            const int idx = it * NT + tid;
            const int tt = idx / (N / 4), e0 = (idx % (N / 4)) * 4;
            if (idx >= RB_TB * (N / 4) || tt >= nt) continue;
            *reinterpret_cast<float4_t*>(&stage[Q_A][tt][e0]) = as_float(raw[it][0]);
            *reinterpret_cast<float4_t*>(&stage[Q_B][tt][e0]) = as_float(raw[it][1]);
            *reinterpret_cast<float4_t*>(&stage[Q_K][tt][e0]) = as_float(raw[it][2]);
            *reinterpret_cast<float4_t*>(&stage[Q_V][tt][e0]) = as_float(raw[it][3]);
            const float4_t w4 = as_float(raw[it][4]);
            float4_t dd, df;
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                const float ew = __expf(w4[m]);
                dd[m] = __expf(-ew);
                df[m] = -ew * dd[m];
            }
            *reinterpret_cast<float4_t*>(&stage[Q_D][tt][e0]) = dd;
            if (reverse_pass) {
                *reinterpret_cast<float4_t*>(&stage[Q_DF][tt][e0]) = df;
                *reinterpret_cast<float4_t*>(&stage[Q_R][tt][e0]) = as_float(raw[it][5]);
                *reinterpret_cast<float4_t*>(&stage[Q_DO][tt][e0]) =
                    d_o != nullptr ? as_float(raw[it][6]) : float4_t{0.f, 0.f, 0.f, 0.f};
            }
        }
    };
    auto block_len = [](int slen, int t0) { return slen - t0 < RB_TB ? slen - t0 : RB_TB; };
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

    if (nseg > 0) request((nseg - 1) * SEG, block_len(T_len - (nseg - 1) * SEG, 0), false);
    for (int seg = nseg - 1; seg >= 0; --seg) {
        const int s0 = seg * SEG;
        const int slen = T_len - s0 < SEG ? T_len - s0 : SEG;
        const int nblk = (slen + RB_TB - 1) / RB_TB;
        // ---- the segment forward once more: the state before each token -> scratch, sa -> LDS
        {
            float4_t s[ROWS];
            const float* src = my_ckpt + (int64_t)seg * ckpt_stride + tile;
#pragma unroll
            for (int i = 0; i < ROWS; ++i) s[i] = *reinterpret_cast<const float4_t*>(src + i * N);
            for (int t0 = 0; t0 < slen; t0 += RB_TB) {
                const int nt = slen - t0 < RB_TB ? slen - t0 : RB_TB;
                __syncthreads();                 // the block before this one has been consumed
                deposit(nt, false);
                __syncthreads();
                if (t0 + RB_TB < slen) request(s0 + t0 + RB_TB, block_len(slen, t0 + RB_TB), false);
                else request(s0 + t0, nt, true);                       // the walk back starts with this block
#pragma unroll 4
                for (int tt = 0; tt < nt; ++tt) {
                    float av[ROWS], d[ROWS], bv[ROWS], kv[ROWS];
                    rows_of(Q_A, tt, av); rows_of(Q_D, tt, d); rows_of(Q_B, tt, bv); rows_of(Q_K, tt, kv);
                    const float4_t v4 = cols_of(Q_V, tt);
                    float4_t sa = {0.f, 0.f, 0.f, 0.f};
                    if (KEEP == 1 || tt % KEEP == 0) {
                        float* dst = my_scr + (int64_t)((t0 + tt) / KEEP) * (N * N) + tile;
#pragma unroll
                        for (int i = 0; i < ROWS; ++i) *reinterpret_cast<float4_t*>(dst + i * N) = s[i];
                    }
#pragma unroll
                    for (int i = 0; i < ROWS; ++i) sa += av[i] * s[i];
                    reduce_rows4<VQ>(sa);
                    if (ks == 0) *reinterpret_cast<float4_t*>(&sa_buf[t0 + tt][col0]) = sa;
#pragma unroll
                    for (int i = 0; i < ROWS; ++i) s[i] = d[i] * s[i] + bv[i] * sa + kv[i] * v4;
                }
            }
        }
        // ---- the segment backwards, block by block (the last, possibly short, block first).  A lane reads back
        // the kept states that it wrote itself, each one group ahead of its use.
        float4_t hk[ROWS];
        auto fetch_kept = [&](int t) {
            const float* src = my_scr + (int64_t)(t / KEEP) * (N * N) + tile;
#pragma unroll
            for (int i = 0; i < ROWS; ++i) hk[i] = *reinterpret_cast<const float4_t*>(src + i * N);
        };
        fetch_kept((slen - 1) / KEEP * KEEP);
        for (int blk = nblk - 1; blk >= 0; --blk) {
            const int t0 = blk * RB_TB;
            const int nt = slen - t0 < RB_TB ? slen - t0 : RB_TB;
            __syncthreads();                     // the block before: vectors consumed, partial sums written out;
                                                 // first block of the segment: the scratch stores above are done
            deposit(nt, true);
            __syncthreads();
            if (blk > 0) request(s0 + t0 - RB_TB, RB_TB, true);
            else if (seg > 0) request(s0 - SEG, RB_TB, false);          // the segment before this one: its first block
            // one token backwards; hp: the state before it
            auto reverse_step = [&](int tt, const float4_t (&hp)[ROWS]) {
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
                const float dv1 = reduce_rows4_scattered<VQ>(dv4);     // row r of the wave: column col0 + r
                reduce_rows4<VQ>(dsa4);
                if ((lane & 15) < VQ)
                    Io<T>::store1(dv + base + (int64_t)(s0 + t0 + tt) * step + col0 + (lane >> 4), dv1);
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
            };
            // a group of KEEP tokens (whole: without a branch between its steps), the last token first
            auto walk_group = [&](int tg, int ng, auto whole) {
                constexpr bool WHOLE = decltype(whole)::value;
                float4_t hs[KEEP][ROWS];         // the states before the group's tokens: the first was kept
#pragma unroll
                for (int i = 0; i < ROWS; ++i) hs[0][i] = hk[i];
                if (t0 + tg >= KEEP) fetch_kept(t0 + tg - KEEP);         // the group before, one group ahead
#pragma unroll
                for (int j = 1; j < KEEP; ++j) {
                    if (!WHOLE && j >= ng) break;
                    float d[ROWS], bv[ROWS], kv[ROWS];
                    rows_of(Q_D, tg + j - 1, d); rows_of(Q_B, tg + j - 1, bv); rows_of(Q_K, tg + j - 1, kv);
                    const float4_t v4 = cols_of(Q_V, tg + j - 1);
                    const float4_t sa4 = *reinterpret_cast<const float4_t*>(&sa_buf[t0 + tg + j - 1][col0]);
#pragma unroll
                    for (int i = 0; i < ROWS; ++i) hs[j][i] = d[i] * hs[j - 1][i] + bv[i] * sa4 + kv[i] * v4;
                }
#pragma unroll
                for (int j = KEEP - 1; j >= 0; --j)
                    if (WHOLE || j < ng) reverse_step(tg + j, hs[j]);
            };
            for (int grp = (nt - 1) / KEEP; grp >= 0; --grp) {
                const int tg = grp * KEEP;
                if (nt - tg >= KEEP) walk_group(tg, KEEP, std::true_type{});
                else walk_group(tg, nt - tg, std::false_type{});
            }
            __syncthreads();
            // the five output rows of the block's tokens: sum over the waves, four channels of one output per thread
            for (int idx = tid; idx < O_COUNT * nt * (N / 4); idx += NT) {
                const int q = idx / (nt * (N / 4)), rem = idx % (nt * (N / 4));
                const int tt = rem / (N / 4), e0 = (rem % (N / 4)) * 4;
                const int64_t off = base + (int64_t)(s0 + t0 + tt) * step + e0;
                float4_t sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int p = 0; p < PARTS; ++p) sum += *reinterpret_cast<const float4_t*>(&part[q][tt][p][e0]);
                if (q == O_DD) sum = sum * *reinterpret_cast<const float4_t*>(&stage[Q_DF][tt][e0]);
                if constexpr (VS > 1) {
                    const int64_t all = (int64_t)(n_bh / H) * T_rows * step;           // elements of one tensor
                    *reinterpret_cast<float4_t*>(pbuf + ((int64_t)vs * O_COUNT + q) * all + off) = sum;
                } else {
                    T* const out = q == O_DR ? dr : q == O_DK ? dk : q == O_DB ? db : q == O_DD ? dw : da;
                    const float o4[4] = {sum.x, sum.y, sum.z, sum.w};
                    Io<T>::store4(out + off, o4);
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
template <int N, int VS, int W> constexpr size_t rec_lds_bytes() {
    typedef RecShape<N, VS, W> Shape;
    return sizeof(float) * ((size_t)8 * Shape::RB * N + (size_t)Shape::SEG * N + (size_t)5 * Shape::RB * W * N);
}

template <typename T, int N, int VS = 1, int W = 4>
hipError_t launch_bwd_rec_t(const BwdArgs& p, const float* ckpt, float* scratch, hipStream_t stream,
                            int ckpt_per_head = 0, int ckpt_step = 1, const int* run_if_any = nullptr, int n_flags = 0,
                            int max_grid = 0, int cu_shift = 4, float* pbuf = nullptr) {
    if (ckpt_per_head == 0) ckpt_per_head = (p.T + RecShape<N>::SEG - 1) / RecShape<N>::SEG;
    const int n_bh = p.B * p.H;
    const int grid = max_grid > 0 && n_bh > max_grid ? max_grid : n_bh * VS;
    constexpr size_t lds = rec_lds_bytes<N, VS, W>();
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(bwd_recurrent_kernel<T, N, VS, W>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    bwd_recurrent_kernel<T, N, VS, W><<<dim3((unsigned)grid), dim3(64 * W), lds, stream>>>(
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
        float* pbuf = scratch + (size_t)p.B * p.H * seg * N * N;
        return p.dtype == RWKV7_DTYPE_BF16  ? launch_bwd_rec_t<bf16_t, 128, 2, W_SPLIT>(p, ckpt, scratch, stream, 0, 1, nullptr, 0, 0, shift, pbuf)
               : p.dtype == RWKV7_DTYPE_F16 ? launch_bwd_rec_t<f16_t, 128, 2, W_SPLIT>(p, ckpt, scratch, stream, 0, 1, nullptr, 0, 0, shift, pbuf)
                                            : launch_bwd_rec_t<float, 128, 2, W_SPLIT>(p, ckpt, scratch, stream, 0, 1, nullptr, 0, 0, shift, pbuf);
    }
    if (N == 128)
        return p.dtype == RWKV7_DTYPE_BF16  ? launch_bwd_rec_t<bf16_t, 128, 1, W_128>(p, ckpt, scratch, stream, 0, 1, nullptr, 0, grid, shift)
               : p.dtype == RWKV7_DTYPE_F16 ? launch_bwd_rec_t<f16_t, 128, 1, W_128>(p, ckpt, scratch, stream, 0, 1, nullptr, 0, grid, shift)
                                            : launch_bwd_rec_t<float, 128, 1, W_128>(p, ckpt, scratch, stream, 0, 1, nullptr, 0, grid, shift);
    return p.dtype == RWKV7_DTYPE_BF16  ? launch_bwd_rec_t<bf16_t, 64, 1, W_64>(p, ckpt, scratch, stream, 0, 1, nullptr, 0, grid, shift)
           : p.dtype == RWKV7_DTYPE_F16 ? launch_bwd_rec_t<f16_t, 64, 1, W_64>(p, ckpt, scratch, stream, 0, 1, nullptr, 0, grid, shift)
                                        : launch_bwd_rec_t<float, 64, 1, W_64>(p, ckpt, scratch, stream, 0, 1, nullptr, 0, grid, shift);
}

}  // namespace rwkv7
