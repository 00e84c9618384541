// Chunked float32 backward of the RWKV7 generalized delta rule for gfx950 (float32 tensors, K = V = 64, dense
// batches): the gradients of the reference's native loop (/root/reference/rwkv_ops/rwkv7_kernel/native_keras_op.py:80-88,
// which the reference differentiates with the host framework's autograd) from the chunk algebra of
// rwkv7_fwd_chunk_f32.hip on chunks of sixteen tokens, every product on the float32 matrix cores.
//
// Per chunk, with h the state before it, dh the adjoint of the state after it and the forward's operands
// (qg, ag, kt, bt, kg, bg, Aqk, Aqb, Aak, N, M = (I - N)^-1, Y = ag h + Aak V, SA = M Y):
//     dSA = Aqb^T dO + bg dh            dY = M^T dSA          dV = Aqk^T dO + kg dh + Aak^T dY
//     dh <- diag(e^G) dh + qg^T dO + ag^T dY                                         (the adjoint of h)
//     dAqk = tril(dO V^T), dAqb = tril(dO SA^T), dAak = tril_-1(dY V^T), dAab = tril_-1(dY SA^T)
//     dqg = dO h^T + dAqk kt + dAqb bt         dag = dY h^T + dAak kt + dAab bt
//     dkt = dAqk^T qg + dAak^T ag              dbt = dAqb^T qg + dAab^T ag
//     dkg = V dh^T                             dbg = SA dh^T
//     dr = dqg e^{gi}, da = dag e^{ge}, dk = dkt e^{-gi} + dkg e^{G-gi}, db = dbt e^{-gi} + dbg e^{G-gi}
//     d(gi) = dqg qg - dkt kt - dbt bt - dkg kg - dbg bg,  d(ge) = dag ag,
//     dG = sum_t (dkg kg + dbg bg) + e^G rowsum(h * dh)
//     dg_t = sum_{s >= t} d(gi)_s + sum_{s > t} d(ge)_s + dG,   dw = dg * (-exp(w))
// Three launches after the forward pass that stores the state before every chunk
// (launch_fwd_chunk_f32_states):
//   1. chunk16_f32_bwd_chain_kernel, one workgroup per (batch, head), chunks last to first: everything the chain of
//      adjoint states runs through (dSA, dY, the new dh) and what has the same shape (Y, SA, dV), with dh before
//      every chunk and SA, dY of every chunk left in the workspace;
//   2. chunk16_f32_bwd_grad_kernel, one workgroup per (batch, head, chunk), no chain: the dA matrices and the six
//      gradients that are [token][key channel];
// A chunk whose decay is too strong for k e^{-gi} (never with RWKV7's own parameterisation) has no chunk form
// here: the forward pass leaves a flag per (batch, head), and when any is set the first kernel returns at once,
// the second stores nothing, and
//   3. the token-by-token kernel of rwkv7_bwd_recurrent.hip, which otherwise returns at once, does the whole call.
#include "rwkv7_f32_mma.h"
#include "rwkv7_kernels.h"
#include "../../include/rwkv7_mi355x.h"

namespace rwkv7 {

namespace {

// ---- chain kernel: one buffer = what the chain waves need of one chunk; three buffers
constexpr int B_QG = 0, B_AG = TILE_F, B_KT = 2 * TILE_F, B_BT = 3 * TILE_F, B_KG = 4 * TILE_F, B_BG = 5 * TILE_F;
constexpr int B_V = 6 * TILE_F, B_DO = 7 * TILE_F;                       // all row-major [token][channel]
// six 1 KiB mailboxes, one float4 per lane
constexpr int B_BOX = 8 * TILE_F;
enum { BOX_AAK_T = 0, BOX_M_T, BOX_AQB, BOX_M, BOX_AQK, BOX_AAK, BOX_COUNT };
constexpr int B_EG = B_BOX + BOX_COUNT * 1024;                           // float [64]: e^G per key channel
constexpr int B_SCR = B_EG + 256;                                        // 1 KiB: the inverting wave transposes N here
constexpr int BBUF = B_SCR + 1024;
constexpr int B_STAGE = 3 * BBUF;                                        // per chain wave: a staging area for its part of a state
constexpr int LDS_CHAIN_BYTES = B_STAGE + 4 * STAGE_BYTES;
static_assert(LDS_CHAIN_BYTES <= 160 * 1024, "one workgroup per CU");

// one float of a row-major tile
__device__ __forceinline__ float tile1(const unsigned char* smem, int off, int row, int col) {
    return *reinterpret_cast<const float*>(smem + off + (row * LDF + col) * 4);
}

// true when any (batch, head) of the call met a chunk with too strong a decay (the forward pass's flags)
__device__ __forceinline__ bool any_strong(const int* __restrict__ flags, int n) {
    int mine = 0;
    for (int i = threadIdx.x; i < n; i += blockDim.x) mine |= flags[i];
    return __syncthreads_or(mine) != 0;
}

// the decays of a chunk and its scaled operands for the channels of one lane (four consecutive ones of one token)
struct Scaled {
    float4_t gstep, gi, G;             // base-2 log decays: this step, inclusive cumulative, chunk total
    float4_t qg, ag, kt, bt, kg, bg;
};
__device__ __forceinline__ void scale_inputs(Scaled& s, bool valid, float4_t W4, float4_t R4, float4_t K4,
                                             float4_t A4, float4_t B4) {
    const float vmask = valid ? 1.f : 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        s.gstep[e] = vmask * fmaxf(-LOG2E * ex2(LOG2E * W4[e]), G_MIN2);   // log2 of exp(-exp(w)); rows past the end: 0
        s.gi[e] = row_inclusive_scan(s.gstep[e]);
        s.G[e] = row_sum(s.gstep[e]);
        const float up = ex2(-s.gi[e]), tail = ex2(s.G[e] - s.gi[e]);
        s.qg[e] = R4[e] * ex2(s.gi[e]);
        s.ag[e] = A4[e] * ex2(s.gi[e] - s.gstep[e]);
        s.kt[e] = K4[e] * up;   s.bt[e] = B4[e] * up;
        s.kg[e] = K4[e] * tail; s.bg[e] = B4[e] * tail;
    }
}

}  // namespace

// Twelve waves as in the forward kernel: waves 0-3 walk the chain, wave w owning value columns 16 w .. + 15 of dh;
// waves 4-7 and 8-11 prepare every other chunk each (operand tiles in one round, the intra-chunk matrices in the
// next).  Chunks are taken last to first: position q = 0, 1, .. is chunk NT - 1 - q, in buffer q % 3.
__global__ __launch_bounds__(768)
void chunk16_f32_bwd_chain_kernel(const float* __restrict__ r_, const float* __restrict__ w_, const float* __restrict__ k_,
                                  const float* __restrict__ v_, const float* __restrict__ a_, const float* __restrict__ b_,
                                  const float* __restrict__ do_, const float* __restrict__ dht,
                                  const float* __restrict__ states, const int* __restrict__ strong_flags,
                                  float* __restrict__ dhs, float* __restrict__ sa_ws, float* __restrict__ dy_ws,
                                  float* __restrict__ dv_, float* __restrict__ dh0, SeqLayout L)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_all[];
    const int H = L.H;
    if (any_strong(strong_flags, L.B * H)) return;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int w = wave & 3;
    const bool producer = wave >= 4;
    const int bh = blockIdx.x, hi = bh % H, bi = bh / H;
    const SeqSpan sp = seq_span(L, bi);
    const int T = sp.len, NT = (T + C16 - 1) / C16;
    const int64_t tok0 = sp.tok0;
    const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
    if (NT == 0) {                             // a sequence without tokens: the adjoint passes through
        if (!producer && dh0 != nullptr) {
            const int x = threadIdx.x & 15, g = (threadIdx.x & 63) >> 4;
            float* dst = dh0 + (int64_t)bh * (NH * NH) + 16 * w + x;
            const float* src = dht == nullptr ? nullptr : dht + (int64_t)bh * (NH * NH) + 16 * w + x;
            for (int i = 0; i < 16; ++i) dst[(4 * i + g) * NH] = src ? src[(4 * i + g) * NH] : 0.f;
        }
        return;
    }
    const int ROUNDS = NT + 2;

    if (producer) {
        const int parity = (wave >> 2) - 1;
        struct Inputs { float4_t R4, W4, K4, V4, A4, B4, D4; };
        auto load_chunk = [&](Inputs& in, int q, int ln) {
            const int c = NT - 1 - q;
            const int t = (c < 0 ? 0 : c) * C16 + (ln & 15);
            const int64_t row = ((tok0 + (t < T ? t : T - 1)) * H + hi) * NH + 16 * w + 4 * (ln >> 4);
            in.W4 = *reinterpret_cast<const float4_t*>(w_ + row); in.R4 = *reinterpret_cast<const float4_t*>(r_ + row);
            in.K4 = *reinterpret_cast<const float4_t*>(k_ + row); in.V4 = *reinterpret_cast<const float4_t*>(v_ + row);
            in.A4 = *reinterpret_cast<const float4_t*>(a_ + row); in.B4 = *reinterpret_cast<const float4_t*>(b_ + row);
            in.D4 = do_ != nullptr ? *reinterpret_cast<const float4_t*>(do_ + row) : float4_t{0.f, 0.f, 0.f, 0.f};
        };
        Inputs next;
        load_chunk(next, parity, (int)(threadIdx.x & 63));
        for (int i = 0; i < parity; ++i) __syncthreads();
        int passed = parity;
        for (int q = parity; q < NT; q += 2) {
            int lane = threadIdx.x & 63;
            asm volatile("" : "+v"(lane));
            const int x = lane & 15, g = lane >> 4;
            const int c = NT - 1 - q;
            unsigned char* smem = smem_all + (q % 3) * BBUF;
            const int ch = 16 * w + 4 * g;
            const bool valid = c * C16 + x < T;
            auto put4 = [&](int off, float4_t val) {
                *reinterpret_cast<float4_t*>(smem + off + (x * LDF + ch) * 4) = val;
            };
            // ---------------------------------------------------------------- round q: the operand tiles
            Inputs cur = next;
            load_chunk(next, q + 2, lane);
            if (!valid) { cur.R4 = cur.K4 = cur.V4 = cur.A4 = cur.B4 = cur.D4 = zero4; }
            {
                Scaled s;
                scale_inputs(s, valid, cur.W4, cur.R4, cur.K4, cur.A4, cur.B4);
                if (x == 0)
                    *reinterpret_cast<float4_t*>(smem + B_EG + ch * 4) = float4_t{ex2(s.G[0]), ex2(s.G[1]), ex2(s.G[2]), ex2(s.G[3])};
                put4(B_QG, s.qg); put4(B_AG, s.ag); put4(B_KT, s.kt); put4(B_BT, s.bt);
                put4(B_KG, s.kg); put4(B_BG, s.bg); put4(B_V, cur.V4); put4(B_DO, cur.D4);
            }
            __syncthreads();
            // ---------------------------------------------------------------- round q + 1: the matrices
            // gram(X, Y): lane (x, g) gets sum_c X[4 g + e][c] Y[x][c]
            auto gram = [&](int off_x, int off_y) {
                float4_t acc = zero4;
#pragma unroll
                for (int ct = 0; ct < 4; ++ct) {
                    const float4_t ax = tile4(smem, off_x, x, 16 * ct + 4 * g);
                    const float4_t by = tile4(smem, off_y, x, 16 * ct + 4 * g);
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc = mfma_f32(ax[e], by[e], acc);
                }
                return acc;
            };
            auto post = [&](int box, float4_t val) {
                *reinterpret_cast<float4_t*>(smem + B_BOX + box * 1024 + lane * 16) = val;
            };
            // R(Z): lane (x, g) holds Z[4 g + e][x];  R(Z^T): Z[x][4 g + e].  For A[i][j] = X_i . Y_j:
            //   R(A)   = gram(X, Y) (row i = 4 g + e, column j = x),  R(A^T) = gram(Y, X) (row i = x, column j = 4 g + e)
            if (w == 0) {
                float4_t acc = gram(B_QG, B_KT);                                 // R(Aqk), j <= i
#pragma unroll
                for (int e = 0; e < 4; ++e) if (x > 4 * g + e) acc[e] = 0.f;
                post(BOX_AQK, acc);
            } else if (w == 3) {
                float4_t acc = gram(B_QG, B_BT);                                 // R(Aqb), j <= i
#pragma unroll
                for (int e = 0; e < 4; ++e) if (x > 4 * g + e) acc[e] = 0.f;
                post(BOX_AQB, acc);
            } else if (w == 1) {
                float4_t acc = gram(B_AG, B_KT);                                 // R(Aak), j < i
#pragma unroll
                for (int e = 0; e < 4; ++e) if (x >= 4 * g + e) acc[e] = 0.f;
                post(BOX_AAK, acc);
                acc = gram(B_KT, B_AG);                                          // R(Aak^T): row i = x, column j = 4 g + e
#pragma unroll
                for (int e = 0; e < 4; ++e) if (4 * g + e >= x) acc[e] = 0.f;
                post(BOX_AAK_T, acc);
            } else {
                // N = tril_-1(ag bt^T), M = (I - N)^-1 = (I + N)(I + N^2)(I + N^4)(I + N^8), both M and M^T
                float4_t NT_ = gram(B_BT, B_AG);                                 // R(N^T): N[x][4 g + e]
#pragma unroll
                for (int e = 0; e < 4; ++e) if (4 * g + e >= x) NT_[e] = 0.f;
                float4_t Nm;                                                     // R(N), through this wave's kilobyte
                {
                    float* scr = reinterpret_cast<float*>(smem + B_SCR);
                    *reinterpret_cast<float4_t*>(scr + x * 16 + 4 * g) = NT_;
#pragma unroll
                    for (int e = 0; e < 4; ++e) Nm[e] = scr[(4 * g + e) * 16 + x];
                }
                float4_t MT = NT_, M_ = Nm;
#pragma unroll
                for (int e = 0; e < 4; ++e) if (4 * g + e == x) { MT[e] += 1.f; M_[e] += 1.f; }
                float4_t P = Nm, PT = NT_;
#pragma unroll
                for (int it = 0; it < 3; ++it) {
                    float4_t P2 = zero4, P2T = zero4;
#pragma unroll
                    for (int e = 0; e < 4; ++e) P2 = mfma_f32(PT[e], P[e], P2);            // R(P P)
                    if (it < 2) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) P2T = mfma_f32(P[e], PT[e], P2T);      // R(P^T P^T)
                    }
                    P = P2; PT = P2T;
                    // D <- D (I + P):  R(D) += mfma(A = R(D^T), B = R(P)),  R(D^T) += mfma(A = R(P), B = R(D^T))
                    float4_t m2 = M_, mt2 = MT;
#pragma unroll
                    for (int e = 0; e < 4; ++e) m2 = mfma_f32(MT[e], P[e], m2);
#pragma unroll
                    for (int e = 0; e < 4; ++e) mt2 = mfma_f32(P[e], MT[e], mt2);
                    M_ = m2; MT = mt2;
                }
                post(BOX_M, M_);
                post(BOX_M_T, MT);
            }
            __syncthreads();
            passed += 2;
        }
        for (; passed < ROUNDS; ++passed) __syncthreads();
        return;
    }

    // ====================================================================== the chain
    // dh: tile ct = rows 16 ct + 4 g + e of column 16 w + x (the forward kernel's layout of the state)
    float4_t dh[4], hn[4];                     // hn: the state before the next chunk, on its way (as it is requested)
    const ChunkRecords record = f32_chunk_records(L, sp, bi, hi, NT);
    float* stage = reinterpret_cast<float*>(smem_all + B_STAGE + w * STAGE_BYTES);
    auto load_state = [&](float4_t (&dst)[4], int c, int ln) {
        state_cols_request(dst, states + record(c < 0 ? 0 : c) * (NH * NH) + 16 * w, ln);
    };
    {
        const int x = threadIdx.x & 15, g = (threadIdx.x & 63) >> 4;
        if (dht != nullptr) {
            const float* src = dht + (int64_t)bh * (NH * NH) + 16 * w + x;
#pragma unroll
            for (int ct = 0; ct < 4; ++ct)
#pragma unroll
                for (int e = 0; e < 4; ++e) dh[ct][e] = src[(16 * ct + 4 * g + e) * NH];
        } else {
#pragma unroll
            for (int ct = 0; ct < 4; ++ct) dh[ct] = zero4;
        }
        load_state(hn, NT - 1, (int)(threadIdx.x & 63));
    }
    __syncthreads();
    __syncthreads();
    for (int q = 0; q < NT; ++q) {
        int lane = threadIdx.x & 63;
        asm volatile("" : "+v"(lane));
        const int x = lane & 15, g = lane >> 4;
        const int c = NT - 1 - q;
        const unsigned char* smem = smem_all + (q % 3) * BBUF;
        const bool valid = c * C16 + x < T;
        // dh after this chunk, for the gradient kernel: row-major [key][value]
        state_cols_store(dhs + record(c) * (NH * NH) + 16 * w, dh, stage, lane);
        float4_t h[4];
        state_cols_unpack(h, hn, stage, lane);
        load_state(hn, c - 1, lane);           // (before the first chunk: that chunk again, never used)

        auto box = [&](int i) { return *reinterpret_cast<const float4_t*>(smem + B_BOX + i * 1024 + lane * 16); };
        const float4_t AakT = box(BOX_AAK_T), MT = box(BOX_M_T), Aqb = box(BOX_AQB), Mm = box(BOX_M),
                       Aqk = box(BOX_AQK), Aak = box(BOX_AAK);
        // Vg[e] = V[token 4 g + e][16 w + x], dOg likewise
        float4_t Vg, dOg;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            Vg[e] = tile1(smem, B_V, 4 * g + e, 16 * w + x);
            dOg[e] = tile1(smem, B_DO, 4 * g + e, 16 * w + x);
        }
        // R(Y) = ag h + Aak V and R(dSA) = Aqb^T dO + bg dh: two independent chains, issued alternately
        float4_t Y = zero4, dSA = zero4;
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
            const float4_t af = tile4(smem, B_AG, x, 16 * ct + 4 * g);
            const float4_t bf = tile4(smem, B_BG, x, 16 * ct + 4 * g);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                Y = mfma_f32(af[e], h[ct][e], Y);
                dSA = mfma_f32(bf[e], dh[ct][e], dSA);
            }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            Y = mfma_f32(AakT[e], Vg[e], Y);
            dSA = mfma_f32(Aqb[e], dOg[e], dSA);
        }
        // R(dY) = M^T dSA;  R(SA^T) = Y^T M^T (lane = token x, values 16 w + 4 g + e: sixteen bytes of one row)
        float4_t dY = zero4, SAT = zero4;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            dY = mfma_f32(Mm[e], dSA[e], dY);
            SAT = mfma_f32(Y[e], MT[e], SAT);
        }
        // R(dV^T) = dO^T Aqk + dh^T kg^T + dY^T Aak,  R(dY^T) = dSA^T M
        float4_t dVT = zero4, dYT = zero4;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            dVT = mfma_f32(dOg[e], Aqk[e], dVT);
            dYT = mfma_f32(dSA[e], Mm[e], dYT);
        }
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
            const float4_t kf = tile4(smem, B_KG, x, 16 * ct + 4 * g);
#pragma unroll
            for (int e = 0; e < 4; ++e) dVT = mfma_f32(dh[ct][e], kf[e], dVT);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) dVT = mfma_f32(dY[e], Aak[e], dVT);
        // dh <- diag(e^G) dh + qg^T dO + ag^T dY: the A operand is qg[token 4 g + e][channel 16 ct + x]
        {
            const float* eg = reinterpret_cast<const float*>(smem + B_EG);
#pragma unroll
            for (int ct = 0; ct < 4; ++ct) dh[ct] = *reinterpret_cast<const float4_t*>(eg + 16 * ct + 4 * g) * dh[ct];
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int ct = 0; ct < 4; ++ct)
                    dh[ct] = mfma_f32(tile1(smem, B_QG, 4 * g + e, 16 * ct + x), dOg[e], dh[ct]);
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int ct = 0; ct < 4; ++ct)
                    dh[ct] = mfma_f32(tile1(smem, B_AG, 4 * g + e, 16 * ct + x), dY[e], dh[ct]);
        }
        {
            const int64_t rec = record(c);
            *reinterpret_cast<float4_t*>(sa_ws + rec * (C16 * NH) + x * NH + 16 * w + 4 * g) = SAT;
            *reinterpret_cast<float4_t*>(dy_ws + rec * (C16 * NH) + x * NH + 16 * w + 4 * g) = dYT;
            if (valid)
                *reinterpret_cast<float4_t*>(dv_ + ((tok0 + c * C16 + x) * H + hi) * NH + 16 * w + 4 * g) = dVT;
        }
        __syncthreads();
    }
    if (dh0 != nullptr) {
        const int x = threadIdx.x & 15, g = (threadIdx.x & 63) >> 4;
        float* dst = dh0 + (int64_t)bh * (NH * NH) + 16 * w + x;
#pragma unroll
        for (int ct = 0; ct < 4; ++ct)
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[(16 * ct + 4 * g + e) * NH] = dh[ct][e];
    }
}

namespace {
// ---- gradient kernel: LDS
constexpr int G_BOX = 0;                       // eight 1 KiB mailboxes: the four dA matrices, each as R(dA^T) and R(dA)
constexpr int LDX = 20;                        // row stride (floats) of a wave's 16 x 16 transposition areas
constexpr int G_TR = G_BOX + 8 * 1024;         // per wave four areas [16 tokens][LDX]
constexpr int TR_BYTES = 16 * LDX * 4;
constexpr int G_HD = G_TR + 4 * 4 * TR_BYTES;  // per wave float [16]
constexpr int G_V = G_HD + 4 * 64, G_DO = G_V + TILE_F, G_SA = G_DO + TILE_F, G_DY = G_SA + TILE_F;   // row-major tiles
constexpr int G_OUT5 = G_DY + TILE_F;           // a fifth tile: the results leave through the four above and this one
constexpr int LDS_GRAD_BYTES = G_OUT5 + TILE_F;
}  // namespace

// One workgroup of four waves per (batch, head, chunk); wave w owns key channels 16 w .. + 15, lane (x, g) token x
// and channels 16 w + 4 g .. + 3 -- the layout of the loads, of the six results (the products are taken
// transposed, R(dX^T): channel 4 g + e, token x) and of the stores.
__global__ __launch_bounds__(256, 2)
void chunk16_f32_bwd_grad_kernel(const float* __restrict__ r_, const float* __restrict__ w_, const float* __restrict__ k_,
                                 const float* __restrict__ v_, const float* __restrict__ a_, const float* __restrict__ b_,
                                 const float* __restrict__ do_, const float* __restrict__ states,
                                 const int* __restrict__ strong_flags, const float* __restrict__ dhs,
                                 const float* __restrict__ sa_ws, const float* __restrict__ dy_ws,
                                 float* __restrict__ dr_, float* __restrict__ dw_, float* __restrict__ dk_,
                                 float* __restrict__ da_, float* __restrict__ db_, SeqLayout L)
{
    __shared__ __attribute__((aligned(16))) unsigned char smem[LDS_GRAD_BYTES];
    // (the forward pass's flags are asked for now and looked at only before the stores: nothing here waits for them)
    const int H = L.H;
    int flagged = 0;
    for (int i = threadIdx.x; i < L.B * H; i += 256) flagged |= strong_flags[i];
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int x = lane & 15, g = lane >> 4;
    int c, bi, hi;
    if (L.cu == nullptr) {                     // dense: workgroup (b H + h) NT + c
        const int nt = (L.T + C16 - 1) / C16;
        c = blockIdx.x % nt;
        const int bh = blockIdx.x / nt;
        hi = bh % H; bi = bh / H;
    } else {
        // packed: workgroup slot H + h; the slot's sequence is the last one that starts at or before it (slots of a
        // sequence start at (first row / 16) + its index, which grows with the index), found by bisection
        const int slot = blockIdx.x / H;
        hi = blockIdx.x % H;
        int lo = 0, up = L.B - 1;
        while (lo < up) {
            const int mid = (lo + up + 1) >> 1;
            if ((int)(seq_span(L, mid).tok0 >> 4) + mid <= slot) lo = mid; else up = mid - 1;
        }
        bi = lo;
        c = slot - ((int)(seq_span(L, bi).tok0 >> 4) + bi);
    }
    const SeqSpan sp = seq_span(L, bi);
    const int T = sp.len, NT = (T + C16 - 1) / C16;
    if (c < 0 || c >= NT) return;              // (packed: a slot between two sequences)
    const int64_t rec = f32_chunk_records(L, sp, bi, hi, NT)(c);
    const int t = c * C16 + x;
    const bool valid = t < T;
    const int64_t row = ((sp.tok0 + (valid ? t : T - 1)) * H + hi) * NH;
    const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};

    // ---- this wave's channels of the inputs, scaled, and four of the scaled operands transposed:
    // T(X)[e] = X[token 4 g + e][channel 16 w + x]
    const int ch = 16 * w + 4 * g;
    float4_t W4 = *reinterpret_cast<const float4_t*>(w_ + row + ch), R4 = *reinterpret_cast<const float4_t*>(r_ + row + ch);
    float4_t K4 = *reinterpret_cast<const float4_t*>(k_ + row + ch), A4 = *reinterpret_cast<const float4_t*>(a_ + row + ch);
    float4_t B4 = *reinterpret_cast<const float4_t*>(b_ + row + ch);
    // V, dO, SA, dY of the chunk ([token][value], all of which every wave needs: both operands of the dA products and
    // the B operands of the products with h and dh): each wave fetches its sixteen columns, through LDS to all
    float4_t Vq = *reinterpret_cast<const float4_t*>(v_ + row + ch);
    float4_t Dq = do_ != nullptr ? *reinterpret_cast<const float4_t*>(do_ + row + ch) : zero4;
    const float4_t Sq = *reinterpret_cast<const float4_t*>(sa_ws + rec * (C16 * NH) + x * NH + ch);
    const float4_t Yq = *reinterpret_cast<const float4_t*>(dy_ws + rec * (C16 * NH) + x * NH + ch);
    // One slab = thirty-two value columns of h and dh, rows [key channel 16 w + x][16 vt + 4 g .. + 3] for two vt
    // (their A operands): the two 64-byte halves of every 128-byte line are requested back to back, so that the second
    // request finds the first one's miss in flight.  The next slab is on its way while this one is multiplied.
    struct Slab { float4_t h[2], dh[2]; };
    auto load_slab = [&](Slab& sl, int pair) {
        const int64_t at = rec * (NH * NH) + (16 * w + x) * NH + 32 * pair + 4 * g;
        sl.h[0] = *reinterpret_cast<const float4_t*>(states + at); sl.h[1] = *reinterpret_cast<const float4_t*>(states + at + 16);
        sl.dh[0] = *reinterpret_cast<const float4_t*>(dhs + at);   sl.dh[1] = *reinterpret_cast<const float4_t*>(dhs + at + 16);
    };
    Slab nxt;
    load_slab(nxt, 0);
    if (!valid) R4 = K4 = A4 = B4 = zero4;
    Scaled s;
    scale_inputs(s, valid, W4, R4, K4, A4, B4);
    float4_t Tqg, Tag, Tkt, Tbt;
    {
        float* tr = reinterpret_cast<float*>(smem + G_TR + w * 4 * TR_BYTES);
        *reinterpret_cast<float4_t*>(tr + 0 * 16 * LDX + x * LDX + 4 * g) = s.qg;
        *reinterpret_cast<float4_t*>(tr + 1 * 16 * LDX + x * LDX + 4 * g) = s.ag;
        *reinterpret_cast<float4_t*>(tr + 2 * 16 * LDX + x * LDX + 4 * g) = s.kt;
        *reinterpret_cast<float4_t*>(tr + 3 * 16 * LDX + x * LDX + 4 * g) = s.bt;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            Tqg[e] = tr[0 * 16 * LDX + (4 * g + e) * LDX + x];
            Tag[e] = tr[1 * 16 * LDX + (4 * g + e) * LDX + x];
            Tkt[e] = tr[2 * 16 * LDX + (4 * g + e) * LDX + x];
            Tbt[e] = tr[3 * 16 * LDX + (4 * g + e) * LDX + x];
        }
    }

    // ---- the products over the value columns.  The dA matrix of this wave, dA[i][j] = left_i . right_j
    // (0: dAqk = dO V^T, 1: dAqb = dO SA^T, 2: dAak = dY V^T, 3: dAab = dY SA^T), as f1 = R(dA^T) (row i = x, column
    // j = 4 g + e) and f2 = R(dA); and the four products that need no dA, R(dX^T)[channel 4 g + e][token x].
    float4_t f1 = zero4, f2 = zero4, dqg = zero4, dag = zero4, dkg = zero4, dbg = zero4, hdp = zero4;
    {
        if (!valid) Vq = Dq = zero4;               // rows past the end
        auto put4 = [&](int off, float4_t val) { *reinterpret_cast<float4_t*>(smem + off + (x * LDF + ch) * 4) = val; };
        put4(G_V, Vq); put4(G_DO, Dq); put4(G_SA, Sq); put4(G_DY, Yq);
    }
    __syncthreads();
#pragma unroll 1
    for (int pair = 0; pair < 2; ++pair) {
        Slab cur = nxt;
        load_slab(nxt, 1);
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int col = 32 * pair + 16 * half + 4 * g;
            const float4_t V4 = tile4(smem, G_V, x, col), D4 = tile4(smem, G_DO, x, col);
            const float4_t S4 = tile4(smem, G_SA, x, col), Y4 = tile4(smem, G_DY, x, col);
            const float4_t right = (w & 1) ? S4 : V4, left = (w & 2) ? Y4 : D4;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                // gram(X, Y): lane (x, g) gets sum_v X[4 g + e][v] Y[x][v]
                f1 = mfma_f32(right[e], left[e], f1);
                f2 = mfma_f32(left[e], right[e], f2);
                dqg = mfma_f32(cur.h[half][e], D4[e], dqg);              // h dO^T
                dkg = mfma_f32(cur.dh[half][e], V4[e], dkg);             // dh V^T
                dag = mfma_f32(cur.h[half][e], Y4[e], dag);              // h dY^T
                dbg = mfma_f32(cur.dh[half][e], S4[e], dbg);             // dh SA^T
            }
            hdp += cur.h[half] * cur.dh[half];
        }
    }
    {
        const bool strict = w >= 2;                                  // dAak, dAab keep j < i
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int j1 = 4 * g + e, i1 = x;                        // f1: dA[i = x][j = 4 g + e]
            const int i2 = 4 * g + e, j2 = x;                        // f2: dA[i = 4 g + e][j = x]
            if (strict ? j1 >= i1 : j1 > i1) f1[e] = 0.f;
            if (strict ? j2 >= i2 : j2 > i2) f2[e] = 0.f;
        }
        *reinterpret_cast<float4_t*>(smem + G_BOX + (2 * w) * 1024 + lane * 16) = f1;
        *reinterpret_cast<float4_t*>(smem + G_BOX + (2 * w + 1) * 1024 + lane * 16) = f2;
    }
    // rowsum(h * dh) of channel 16 w + x, brought to the lanes that own the channel
    float4_t hd4;
    {
        float hd = (hdp[0] + hdp[1]) + (hdp[2] + hdp[3]);
        hd = sum_over_rows(hd);
        float* hdl = reinterpret_cast<float*>(smem + G_HD + w * 64);
        if (g == 0) hdl[x] = hd;
        hd4 = *reinterpret_cast<const float4_t*>(hdl + 4 * g);
    }
    const bool strong = __syncthreads_or(flagged) != 0;     // then the token-by-token kernel does the whole call
    auto box = [&](int i) { return *reinterpret_cast<const float4_t*>(smem + G_BOX + i * 1024 + lane * 16); };
    float4_t dkt = zero4, dbt = zero4;
    {
        const float4_t dAqk1 = box(0), dAqk2 = box(1), dAqb1 = box(2), dAqb2 = box(3);
        const float4_t dAak1 = box(4), dAak2 = box(5), dAab1 = box(6), dAab2 = box(7);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            dqg = mfma_f32(Tkt[e], dAqk1[e], dqg);                   // kt^T dAqk^T
            dag = mfma_f32(Tkt[e], dAak1[e], dag);                   // kt^T dAak^T
            dkt = mfma_f32(Tqg[e], dAqk2[e], dkt);                   // qg^T dAqk
            dbt = mfma_f32(Tqg[e], dAqb2[e], dbt);                   // qg^T dAqb
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            dqg = mfma_f32(Tbt[e], dAqb1[e], dqg);                   // bt^T dAqb^T
            dag = mfma_f32(Tbt[e], dAab1[e], dag);                   // bt^T dAab^T
            dkt = mfma_f32(Tag[e], dAak2[e], dkt);                   // ag^T dAak
            dbt = mfma_f32(Tag[e], dAab2[e], dbt);                   // ag^T dAab
        }
    }

    // ---- the gradients of the inputs
    float4_t dr, dw, dk, da, db;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float egi = ex2(s.gi[e]), ege = ex2(s.gi[e] - s.gstep[e]), up = ex2(-s.gi[e]), tail = ex2(s.G[e] - s.gi[e]);
        dr[e] = dqg[e] * egi;
        da[e] = dag[e] * ege;
        dk[e] = dkt[e] * up + dkg[e] * tail;
        db[e] = dbt[e] * up + dbg[e] * tail;
        const float end = dkg[e] * s.kg[e] + dbg[e] * s.bg[e];
        const float dgi = dqg[e] * s.qg[e] - dkt[e] * s.kt[e] - dbt[e] * s.bt[e] - end;
        const float dge = dag[e] * s.ag[e];
        const float dG = row_sum(end) + ex2(s.G[e]) * hd4[e];
        // g_t enters gi_s for s >= t, ge_s for s > t, G always
        const float after_gi = row_sum(dgi) - row_inclusive_scan(dgi) + dgi;
        const float after_ge = row_sum(dge) - row_inclusive_scan(dge);
        // d(log decay)/dw = -exp(w), the natural-log decay itself (zero where the clamp holds it)
        const float gnat = s.gstep[e] > G_MIN2 ? s.gstep[e] * (1.f / LOG2E) : 0.f;
        dw[e] = (after_gi + after_ge + dG) * gnat;
    }
    // The results go through LDS so that a wave stores whole 256-byte rows (tokens 4 w .. + 3, lane = sixteen bytes
    // of a row) instead of a 64-byte piece of each of sixteen rows.  (The four tiles of the inputs have been read by
    // everybody before the last barrier.)
    {
        auto put4 = [&](int off, float4_t val) { *reinterpret_cast<float4_t*>(smem + off + (x * LDF + ch) * 4) = val; };
        put4(G_V, dr); put4(G_DO, dw); put4(G_SA, dk); put4(G_DY, da); put4(G_OUT5, db);
    }
    __syncthreads();
    {
        const int tok = 4 * w + g, piece = 4 * x, ts = c * C16 + tok;
        if (ts < T && !strong) {
            const int64_t o = ((sp.tok0 + ts) * H + hi) * NH + piece;
            *reinterpret_cast<float4_t*>(dr_ + o) = tile4(smem, G_V, tok, piece);
            *reinterpret_cast<float4_t*>(dw_ + o) = tile4(smem, G_DO, tok, piece);
            *reinterpret_cast<float4_t*>(dk_ + o) = tile4(smem, G_SA, tok, piece);
            *reinterpret_cast<float4_t*>(da_ + o) = tile4(smem, G_DY, tok, piece);
            *reinterpret_cast<float4_t*>(db_ + o) = tile4(smem, G_OUT5, tok, piece);
        }
    }
}

// Workspace: per record (one per 16-token chunk and head; packed sequences: (T_total / 16 + n_seq) H of them) the state
// before the chunk, dh after it, SA and dY; the token-by-token kernel's scratch areas (64 states each: one per
// (batch, head), at most WALK_MAX_GRID with packed sequences); one flag per (sequence, head).
namespace {
size_t f32_records(int B, int T, int H, bool varlen) {
    return varlen ? ((size_t)(T >> 4) + B) * H : (size_t)B * H * ((T + C16 - 1) / C16);
}
size_t walk_areas(int B, int H, bool varlen) {
    const size_t bh = (size_t)B * H;
    return varlen && bh > (size_t)WALK_MAX_GRID ? (size_t)WALK_MAX_GRID : bh;
}
}  // namespace

size_t bwd_chunk_f32_workspace_bytes(int B, int T, int H, bool varlen) {
    const size_t per_chunk = (size_t)(2 * NH * NH + 2 * C16 * NH) * 4;
    return f32_records(B, T, H, varlen) * per_chunk + walk_areas(B, H, varlen) * 64 * (size_t)(NH * NH) * 4 +
           (((size_t)B * H * 4 + 255) & ~(size_t)255);
}

hipError_t launch_bwd_chunk_f32(const BwdArgs& p, void* ws, hipStream_t stream) {
    const bool varlen = p.cu != nullptr;
    const size_t BH = (size_t)p.B * p.H, NR = f32_records(p.B, p.T, p.H, varlen);
    float* states = static_cast<float*>(ws);
    float* dhs = states + NR * (NH * NH);
    float* sa = dhs + NR * (NH * NH);
    float* dy = sa + NR * (C16 * NH);
    float* scratch = dy + NR * (C16 * NH);
    int* flags = reinterpret_cast<int*>(scratch + walk_areas(p.B, p.H, varlen) * 64 * (size_t)(NH * NH));
    // launch 1: the forward once more, leaving the state before every chunk and the flags
    SeqArgs f{};
    f.r = p.r; f.w = p.w; f.k = p.k; f.v = p.v; f.a = p.a; f.b = p.b;
    f.h0 = p.h0; f.h0_batch_stride = p.h0 ? p.h0_batch_stride : 0;
    f.B = p.B; f.T = p.T; f.H = p.H; f.N = NH; f.dtype = p.dtype; f.cu = p.cu;
    const SeqLayout L = seq_layout(f, nullptr);
    hipError_t e;
    if (varlen) {                      // rows of the gradients behind the last sequence
        TailFill tail;
        tail.p[0] = p.dr; tail.p[1] = p.dw; tail.p[2] = p.dk; tail.p[3] = p.dv; tail.p[4] = p.da; tail.p[5] = p.db;
        tail.n = 6; tail.row_bytes = (int64_t)p.H * NH * 4;
        e = launch_chunk_items(L, nullptr, nullptr, 0, nullptr, tail, stream);
        if (e != hipSuccess) return e;
    }
    e = launch_fwd_chunk_f32_states(f, states, C16, stream, flags);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(chunk16_f32_bwd_chain_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, LDS_CHAIN_BYTES);
    if (e != hipSuccess) return e;
    chunk16_f32_bwd_chain_kernel<<<dim3((unsigned)BH), dim3(768), LDS_CHAIN_BYTES, stream>>>(
        (const float*)p.r, (const float*)p.w, (const float*)p.k, (const float*)p.v, (const float*)p.a,
        (const float*)p.b, (const float*)p.dO, p.dht, states, flags, dhs, sa, dy, (float*)p.dv, p.dh0, L);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    chunk16_f32_bwd_grad_kernel<<<dim3((unsigned)NR), dim3(256), 0, stream>>>(
        (const float*)p.r, (const float*)p.w, (const float*)p.k, (const float*)p.v, (const float*)p.a,
        (const float*)p.b, (const float*)p.dO, states, flags, dhs, sa, dy, (float*)p.dr, (float*)p.dw, (float*)p.dk,
        (float*)p.da, (float*)p.db, L);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    // strong decays somewhere: the two kernels above have returned at once / stored nothing, this one does the call
    return launch_bwd_recurrent_walk_f32(p, states, scratch, flags, (int)BH, stream);
}

}  // namespace rwkv7
