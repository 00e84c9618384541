// Chunked bf16-MFMA forward of the RWKV7 generalized delta rule for head size K = V = 128 on gfx950
// (the head size of /root/reference/test_script/test_rwkv7_value.py:48-53).
//
// The same chunk algebra as the K = 64 kernels (rwkv7_fwd_chunk.hip; the reference's chunk_dplr_fwd,
// /root/reference/rwkv_ops/rwkv7_kernel/torch_op.py:46-120), per 64-token chunk with gi / ge the inclusive /
// exclusive cumulative log decay and G its total:
//     qg = r e^{gi}, ag = a e^{ge}, kt = k e^{-gi}, bt = b e^{-gi}, kg = k e^{G-gi}, bg = b e^{G-gi},
//     Aqk = tril(qg kt^T), Aqb = tril(qg bt^T), Aak = tril_-1(ag kt^T), Aab = tril_-1(ag bt^T), M = (I - Aab)^-1,
//     Y = ag h + Aak V,  SA = M Y,  O = qg h + Aqk V + Aqb SA,  h' = diag(e^G) h + kg^T V + bg^T SA.
// A 128x128 float32 state is 64 KiB, four times the K = 64 one, so the shape of the kernel is different: ONE
// workgroup of eight waves per (batch, head) walks the sequence chunk by chunk with the state in registers
// (wave = 16 value columns, 32 accumulator registers per lane) -- no workspace, no hand-off between workgroups.
// Every operand of a chunk is a row-major bf16 tile in LDS ([64 tokens][128 channels], or 64x64 for the
// intra-chunk matrices), read along its rows or, with ds_read_b64_tr_b16, along its columns; products whose
// result feeds the next product (Y -> SA -> O, h') stay in registers: an accumulator tile pair packed to bf16 IS
// the next B operand in the permuted ("sigma") contraction order of rwkv7_mma.h.  The state enters every product
// as bf16 hi + lo, so it keeps about 16 mantissa bits.  A chunk whose decay is too strong for k e^{-gi} to stay in
// range (never with RWKV7's own decay range) is walked token by token in float32 instead.
#include "rwkv7_chunk.h"
#include "rwkv7_kernels.h"
#include "../../include/rwkv7_mi355x.h"

namespace rwkv7 {

namespace {

constexpr int N128 = 128;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float BUCKET2 = BUCKET * LOG2E;      // exponent range of one decay bucket, in base-2 units
constexpr float G_MIN2 = G_MIN * LOG2E;        // per-step log-decay clamp, in base-2 units
__device__ __forceinline__ float ex2(float x) { return __builtin_amdgcn_exp2f(x); }

constexpr int LDW = 136;                       // row stride (elements) of the [64][128] tiles (144, which would free the
                                               // transposing reads of bank conflicts, costs the row reads more: + 12 %)
constexpr int WT = 64 * LDW * 2;               // bytes of one
constexpr int LDA = LDT;                       // row stride of the 64x64 tiles
constexpr int AT = 64 * LDA * 2;
constexpr int LDO = 72;                        // row stride of the output tile [128 values][64 tokens]
constexpr int OFF_QG = 0, OFF_AG = WT, OFF_KT = 2 * WT, OFF_BT = 3 * WT, OFF_V = 4 * WT;
constexpr int OFF_AQK = 5 * WT, OFF_AQB = OFF_AQK + AT, OFF_AAK = OFF_AQB + AT, OFF_AAB = OFF_AAK + AT,
              OFF_MT = OFF_AAB + AT;
constexpr int OFF_OT = OFF_MT + AT;            // O^T [value][token]
constexpr int OFF_TOT = OFF_OT + N128 * LDO * 2;     // float [4 token tiles][128]: tile totals of the log decay
constexpr int OFF_XM = OFF_TOT + 4 * N128 * 4; // float [8]: per-wave maxima of the chunk's total decay
constexpr int OFF_EG = OFF_XM + 64;            // float [128]: e^G per key channel
constexpr int OFF_DI = OFF_EG + N128 * 4;      // 4 inverted diagonal blocks, bf16 16x16
constexpr int LDS128_BYTES = OFF_DI + 4 * 512;
static_assert(LDS128_BYTES <= 160 * 1024, "one workgroup per CU");

// "plain" A / B fragment of a row-major tile: row 16 rt + x, columns 32 s + 8 g .. + 7
__device__ __forceinline__ bf16x8_t rows_plain(const unsigned char* smem, int off, int ld, int rt, int s, int lane) {
    const int x = lane & 15, g = lane >> 4;
    return *reinterpret_cast<const bf16x8_t*>(smem + off + ((16 * rt + x) * ld + 32 * s + 8 * g) * 2);
}
// "sigma" fragment of a row-major tile: row 16 rt + x, columns 32 s + 4 g .. + 3 and 32 s + 16 + 4 g .. + 3
__device__ __forceinline__ bf16x8_t rows_sigma(const unsigned char* smem, int off, int ld, int rt, int s, int lane) {
    const int x = lane & 15, g = lane >> 4;
    const unsigned char* p = smem + off + ((16 * rt + x) * ld + 32 * s + 4 * g) * 2;
    const bf16x4_t lo = *reinterpret_cast<const bf16x4_t*>(p);
    const bf16x4_t hi = *reinterpret_cast<const bf16x4_t*>(p + 32);
    return bf16x8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}
// accumulator tile (column n = 16 nt + x, rows 16 mt + 4 g .. + 3) -> tile[n][m], an 8-byte store
__device__ __forceinline__ void store_acc_t(unsigned char* smem, int off, int ld, int nt, int mt, int lane, float4_t acc) {
    const int x = lane & 15, g = lane >> 4;
    *reinterpret_cast<bf16x4_t*>(smem + off + ((16 * nt + x) * ld + 16 * mt + 4 * g) * 2) = pack4(acc);
}

}  // namespace

__global__ __launch_bounds__(512, 1)
void chunk128_fwd_kernel(const bf16_t* __restrict__ r_, const bf16_t* __restrict__ w_, const bf16_t* __restrict__ k_,
                         const bf16_t* __restrict__ v_, const bf16_t* __restrict__ a_, const bf16_t* __restrict__ b_,
                         const float* __restrict__ h0, int64_t h0_batch_stride, const int* __restrict__ h0_map,
                         int n_state, bf16_t* __restrict__ o_, float* __restrict__ ht, SeqLayout L)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    constexpr int N = N128;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int w = wv & 3, hf = wv >> 2;        // chunk phases: token tile w, channel half hf
    const int H = L.H;
    const int bh = blockIdx.x, hi = bh % H, bi = bh / H;
    const SeqSpan sp = seq_span(L, bi);
    const int T = sp.len, NT = (T + CH - 1) / CH;
    const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};

    // state: wave wv owns value columns 16 wv .. + 15; tile ct: h[16 ct + 4 g + e][16 wv + x]
    float4_t h[8];
    if (h0 != nullptr) {
        const int x = threadIdx.x & 15, g = (threadIdx.x & 63) >> 4;
        const float* src = h0 + state_row(h0_map, n_state, bi) * h0_batch_stride + (int64_t)hi * (N * N) + 16 * wv + x;
#pragma unroll
        for (int ct = 0; ct < 8; ++ct)
#pragma unroll
            for (int e = 0; e < 4; ++e) h[ct][e] = src[(16 * ct + 4 * g + e) * N];
    } else {
#pragma unroll
        for (int ct = 0; ct < 8; ++ct) h[ct] = zero4;
    }

    bf16x8_t R[2], W[2], K[2], V[2], A[2], B[2];
    // part: bit 0 = w, r; bit 1 = k, v; bit 2 = a, b.  Inside the loop a chunk's inputs are requested in these three
    // groups, each behind a different product: a wave that issues all twelve requests at once sits at the issue stage
    // until the memory pipeline has taken them.
    auto load_chunk = [&](int c, int ln, int part) {
        const int t = c * CH + 16 * w + (ln & 15);
        const int c0 = 64 * hf + 8 * (ln >> 4), c1 = c0 + 32;
        // rows past the sequence's end (last chunk only) are read from the last valid row and zeroed by the consumer
        const int64_t row = ((sp.tok0 + (t < T ? t : T - 1)) * H + hi) * N;
        if (part & 1) {
            W[0] = *reinterpret_cast<const bf16x8_t*>(w_ + row + c0); W[1] = *reinterpret_cast<const bf16x8_t*>(w_ + row + c1);
            R[0] = *reinterpret_cast<const bf16x8_t*>(r_ + row + c0); R[1] = *reinterpret_cast<const bf16x8_t*>(r_ + row + c1);
        }
        if (part & 2) {
            K[0] = *reinterpret_cast<const bf16x8_t*>(k_ + row + c0); K[1] = *reinterpret_cast<const bf16x8_t*>(k_ + row + c1);
            V[0] = *reinterpret_cast<const bf16x8_t*>(v_ + row + c0); V[1] = *reinterpret_cast<const bf16x8_t*>(v_ + row + c1);
        }
        if (part & 4) {
            A[0] = *reinterpret_cast<const bf16x8_t*>(a_ + row + c0); A[1] = *reinterpret_cast<const bf16x8_t*>(a_ + row + c1);
            B[0] = *reinterpret_cast<const bf16x8_t*>(b_ + row + c0); B[1] = *reinterpret_cast<const bf16x8_t*>(b_ + row + c1);
        }
    };
    if (NT > 0) load_chunk(0, (int)(threadIdx.x & 63), 7);
    for (int c = 0; c < NT; ++c) {
        // The lane id is made opaque per chunk, so that the per-lane addresses are formed where they are used
        // instead of being hoisted out of the loop and kept in (spilled) registers.
        int lane = threadIdx.x & 63;
        asm volatile("" : "+v"(lane));
        const int x = lane & 15, g = lane >> 4;
        const int t_local = 16 * w + x;
        const int c0 = 64 * hf + 8 * g, c1 = c0 + 32;      // this lane's two 8-channel pieces in the load layout
        auto put_row = [&](int off, const bf16x8_t (&f)[2]) {
            *reinterpret_cast<bf16x8_t*>(smem + off + (t_local * LDW + c0) * 2) = f[0];
            *reinterpret_cast<bf16x8_t*>(smem + off + (t_local * LDW + c1) * 2) = f[1];
        };
        // this lane's 16 cumulative log decays of chunk c (base 2, inclusive), the per-step ones and the chunk totals,
        // from the raw w and the tile totals that P0 leaves in LDS
        auto decays = [&](bool valid, float (&gl)[16], float (&gstep)[16], float (&gsum)[16]) {
    #pragma unroll
            for (int e = 0; e < 16; ++e) {
                // log2 of exp(-exp(w)); rows past the end: times zero (a select becomes a branch around each evaluation)
                gstep[e] = (valid ? 1.f : 0.f) * fmaxf(-LOG2E * ex2(LOG2E * (float)W[e >> 3][e & 7]), G_MIN2);
                gl[e] = row_inclusive_scan(gstep[e]);
                if ((e & 3) == 3) __builtin_amdgcn_sched_barrier(0);      // (keeps the sixteen evaluations from being interleaved)
            }
            float* tot = reinterpret_cast<float*>(smem + OFF_TOT);
            if (x == 15) {
    #pragma unroll
                for (int s = 0; s < 2; ++s) {
                    float4_t* dst = reinterpret_cast<float4_t*>(tot + w * N + (s ? c1 : c0));
                    dst[0] = float4_t{gl[8 * s], gl[8 * s + 1], gl[8 * s + 2], gl[8 * s + 3]};
                    dst[1] = float4_t{gl[8 * s + 4], gl[8 * s + 5], gl[8 * s + 6], gl[8 * s + 7]};
                }
            }
            __syncthreads();                                                           // B0
    #pragma unroll
            for (int e = 0; e < 16; ++e) gsum[e] = 0.f;
    #pragma unroll
            for (int ww = 0; ww < 4; ++ww) {
    #pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const float4_t* src = reinterpret_cast<const float4_t*>(tot + ww * N + (s ? c1 : c0));
                    const float4_t a0 = src[0], a1 = src[1];
                    const float vals[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
    #pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        gsum[8 * s + j] += vals[j];
                        if (ww < w) gl[8 * s + j] += vals[j];
                    }
                }
            }
        };
        auto put_piece = [&](int off, int s, const bf16x8_t& f) {
            *reinterpret_cast<bf16x8_t*>(smem + off + (t_local * LDW + (s ? c1 : c0)) * 2) = f;
        };
        // qg = r e^{gi}, ag = a e^{ge}, kt = k e^{-gi}, bt = b e^{-gi} -> their tiles, one 8-channel piece at a time
        auto operand_tiles = [&](const float (&gl)[16], const float (&gstep)[16]) {
    #pragma unroll
            for (int s = 0; s < 2; ++s) {
                bf16x8_t Qp, Ap, Kp, Bp;
    #pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int e = 8 * s + j;
                    const float up = ex2(-gl[e]);
                    Kp[j] = (bf16_t)((float)K[s][j] * up);
                    Bp[j] = (bf16_t)((float)B[s][j] * up);
                    Qp[j] = (bf16_t)((float)R[s][j] * ex2(gl[e]));
                    Ap[j] = (bf16_t)((float)A[s][j] * ex2(gl[e] - gstep[e]));
                }
                put_piece(OFF_QG, s, Qp); put_piece(OFF_AG, s, Ap); put_piece(OFF_KT, s, Kp); put_piece(OFF_BT, s, Bp);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        auto zero_ragged = [&](bool valid, bool ragged) {
            if (ragged && !valid) {
                const bf16x8_t z = zero_frag();
                R[0] = R[1] = K[0] = K[1] = V[0] = V[1] = A[0] = A[1] = B[0] = B[1] = z;
            }
        };

        const bool valid = c * CH + t_local < T;
        const bool ragged = (c + 1) * CH > T;      // uniform: only the last chunk of a sequence can be
        zero_ragged(valid, ragged);
        // ---- P0: cumulative log decays; the scaled operands -> tiles; kg, bg kept packed for later
        bf16x8_t KG[2], BG[2];
        {
            float gl[16], gstep[16], gsum[16];
            decays(valid, gl, gstep, gsum);
            float xmax = 0.f;
#pragma unroll
            for (int e = 0; e < 16; ++e) xmax = fmaxf(xmax, -gsum[e]);
            xmax = max_over_rows(xmax);
            if (lane == 0) reinterpret_cast<float*>(smem + OFF_XM)[wv] = xmax;
            if (w == 0 && x == 0) {        // decay of the whole chunk per key channel
                float* eg = reinterpret_cast<float*>(smem + OFF_EG);
#pragma unroll
                for (int e = 0; e < 16; ++e) eg[(e < 8 ? c0 : c1) + (e & 7)] = ex2(gsum[e]);
            }
            operand_tiles(gl, gstep);
            put_row(OFF_V, V);
#pragma unroll
            for (int e = 0; e < 16; ++e) {         // kg, bg: exponent G - gi <= 0, no buckets
                const int s = e >> 3, j = e & 7;
                const float tail = ex2(gsum[e] - gl[e]);
                KG[s][j] = (bf16_t)((float)K[s][j] * tail);
                BG[s][j] = (bf16_t)((float)B[s][j] * tail);
                if ((e & 3) == 3) __builtin_amdgcn_sched_barrier(0);
            }
        }
        __syncthreads();                                                           // B1
        bool strong;                       // uniform over the workgroup: some channel decays by more than e^-64 over the chunk
        {
            const float* xm = reinterpret_cast<const float*>(smem + OFF_XM);
            float xmax = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) xmax = fmaxf(xmax, xm[i]);
            strong = xmax >= BUCKET2;
        }
        if (strong) {
            // Strong decays (never with RWKV7's own parameterisation, |log decay| <= 0.607 per step): k e^{-gi} would
            // overflow, and rather than accumulate the intra-chunk matrices over exponent buckets as the K = 64
            // kernels do, this chunk is walked token by token in float32 (the arithmetic of the recurrent kernel)
            // on the state as it lies in the registers: lane (x, g) of wave wv holds rows 16 ct + 4 g + e of
            // column 16 wv + x.  The raw inputs replace the scaled operands in their tiles; the decays go to a
            // float32 tile over the (unused) intra-chunk matrices.
            put_row(OFF_QG, R); put_row(OFF_AG, A); put_row(OFF_KT, K); put_row(OFF_BT, B);
            float* dtile = reinterpret_cast<float*>(smem + OFF_AQK);               // [64 tokens][128] float
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                float dv[8];
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    dv[j] = valid ? ex2(fmaxf(-LOG2E * ex2(LOG2E * (float)W[s][j]), G_MIN2)) : 1.f;
                float4_t* dst = reinterpret_cast<float4_t*>(dtile + t_local * N + (s ? c1 : c0));
                dst[0] = float4_t{dv[0], dv[1], dv[2], dv[3]};
                dst[1] = float4_t{dv[4], dv[5], dv[6], dv[7]};
            }
            __syncthreads();
            if (c + 1 < NT) load_chunk(c + 1, lane, 7);
            const int nt = T - c * CH < CH ? T - c * CH : CH;
            for (int tt = 0; tt < nt; ++tt) {
                float4_t sa4 = zero4;          // partial sums over this lane's rows, tile by tile
                const bf16_t vv = *reinterpret_cast<const bf16_t*>(smem + OFF_V + (tt * LDW + 16 * wv + x) * 2);
#pragma unroll
                for (int ct = 0; ct < 8; ++ct) {
                    const float4_t a4 = unpack4(*reinterpret_cast<const bf16x4_t*>(smem + OFF_AG + (tt * LDW + 16 * ct + 4 * g) * 2));
                    sa4 += a4 * h[ct];
                }
                float sa = (sa4.x + sa4.y) + (sa4.z + sa4.w);
                sa = sum_over_rows(sa);
                float4_t o4 = zero4;
                const float vf = (float)vv;
#pragma unroll
                for (int ct = 0; ct < 8; ++ct) {
                    const int col = tt * LDW + 16 * ct + 4 * g;
                    const float4_t d4 = *reinterpret_cast<const float4_t*>(dtile + tt * N + 16 * ct + 4 * g);
                    const float4_t b4 = unpack4(*reinterpret_cast<const bf16x4_t*>(smem + OFF_BT + col * 2));
                    const float4_t k4 = unpack4(*reinterpret_cast<const bf16x4_t*>(smem + OFF_KT + col * 2));
                    const float4_t r4 = unpack4(*reinterpret_cast<const bf16x4_t*>(smem + OFF_QG + col * 2));
                    h[ct] = d4 * h[ct] + b4 * sa + k4 * vf;
                    o4 += r4 * h[ct];
                }
                float ov = (o4.x + o4.y) + (o4.z + o4.w);
                ov = sum_over_rows(ov);
                if (g == 0) o_[((sp.tok0 + c * CH + tt) * H + hi) * N + 16 * wv + x] = (bf16_t)ov;
            }
            __syncthreads();               // the next chunk rewrites the tiles
            continue;
        }

        // ---- P1: block row w (rows j, column i = 16 w + x) of Aqk, Aqb (waves hf = 0) and of Aak, Aab
        // (waves hf = 1); contraction over the 128 channels in four k-steps
        float4_t acc1[4], acc2[4];
        float4_t diagX = zero4;
#pragma unroll
        for (int J = 0; J < 4; ++J) { acc1[J] = zero4; acc2[J] = zero4; }
        {
            const int s_qa = hf ? OFF_AG : OFF_QG;
            bf16x8_t qa[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) qa[s] = rows_plain(smem, s_qa, LDW, w, s, lane);
#pragma unroll
            for (int J = 0; J < 4; ++J) {
                if (J <= w) {
#pragma unroll
                    for (int s = 0; s < 4; ++s) {
                        acc1[J] = mfma_bf16(rows_plain(smem, OFF_KT, LDW, J, s, lane), qa[s], acc1[J]);
                        acc2[J] = mfma_bf16(rows_plain(smem, OFF_BT, LDW, J, s, lane), qa[s], acc2[J]);
                    }
                }
            }
            if (hf) {
#pragma unroll
                for (int s = 0; s < 4; ++s)
                    diagX = mfma_bf16(qa[s], rows_plain(smem, OFF_BT, LDW, w, s, lane), diagX);
            }
        }
        __syncthreads();                   // every read of kt, bt is done: kg, bg take their tiles
        put_row(OFF_KT, KG); put_row(OFF_BT, BG);
        float4_t diagXT = zero4;
#pragma unroll
        for (int J = 0; J < 4; ++J) {
            if (J == w) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int jj = 4 * g + e;
                    // causal masks on the diagonal block: j <= i for Aqk/Aqb, j < i for Aak/Aab
                    if (hf ? jj >= x : jj > x) { acc1[J][e] = 0.f; acc2[J][e] = 0.f; }
                    if (x >= jj) diagX[e] = 0.f;
                }
                diagXT = acc2[J];
            }
            // tiles [i][j]: row i = 16 w + x, columns 16 J + 4 g .. + 3 (zero right of the diagonal block)
            store_acc_t(smem, hf ? OFF_AAK : OFF_AQK, LDA, w, J, lane, J <= w ? acc1[J] : zero4);
            store_acc_t(smem, hf ? OFF_AAB : OFF_AQB, LDA, w, J, lane, J <= w ? acc2[J] : zero4);
        }
        // inverse of the diagonal block: (I - X)^-1 = (I + X)(I + X^2)(I + X^4)(I + X^8), X strictly lower 16x16;
        // the waves that hold Aab do it
        float4_t Dm = zero4;
        if (hf) {
            float4_t DmT;
            bf16x4_t Pb = pack4(diagX), PbT = pack4(diagXT);
            Dm = diagX; DmT = diagXT;
#pragma unroll
            for (int e = 0; e < 4; ++e) if (4 * g + e == x) { Dm[e] += 1.f; DmT[e] += 1.f; }
#pragma unroll
            for (int it = 0; it < 3; ++it) {
                const float4_t P2 = mfma_bf16_k16(PbT, Pb, zero4);
                const float4_t P2T = mfma_bf16_k16(Pb, PbT, zero4);
                Pb = pack4(P2); PbT = pack4(P2T);
                const bf16x4_t DbT = pack4(DmT);
                Dm = mfma_bf16_k16(DbT, Pb, Dm);
                DmT = mfma_bf16_k16(Pb, DbT, DmT);
            }
            *reinterpret_cast<bf16x4_t*>(smem + OFF_DI + w * 512 + (x * 16 + 4 * g) * 2) = pack4(DmT);
        }
        __syncthreads();
        // M^T tile [j][i]: column block J = w, rows i >= j; zero above the diagonal blocks
        if (hf) {
            store_acc_t(smem, OFF_MT, LDA, w, w, lane, Dm);
#pragma unroll
            for (int I = 0; I < 4; ++I) if (I < w) store_acc_t(smem, OFF_MT, LDA, w, I, lane, zero4);
            bf16x4_t Mcol[4];
            Mcol[0] = Mcol[1] = Mcol[2] = Mcol[3] = pack4(zero4);
#pragma unroll
            for (int Lc = 0; Lc < 4; ++Lc) if (Lc == w) Mcol[Lc] = pack4(Dm);
#pragma unroll
            for (int I = 1; I < 4; ++I) {
                if (I > w) {
                    float4_t S = zero4;
#pragma unroll
                    for (int Lc = 0; Lc < 3; ++Lc) {
                        if (Lc >= w && Lc < I) {
                            const bf16x4_t a4 = *reinterpret_cast<const bf16x4_t*>(
                                smem + OFF_AAB + ((16 * I + x) * LDA + 16 * Lc + 4 * g) * 2);
                            S = mfma_bf16_k16(a4, Mcol[Lc], S);
                        }
                    }
                    const bf16x4_t d4 = *reinterpret_cast<const bf16x4_t*>(smem + OFF_DI + I * 512 + (x * 16 + 4 * g) * 2);
                    const float4_t Mi = mfma_bf16_k16(d4, pack4(S), zero4);
                    Mcol[I] = pack4(Mi);
                    store_acc_t(smem, OFF_MT, LDA, w, I, lane, Mi);     // column j = 16 w + x, rows i = 16 I + 4 g + e
                }
            }
        }
        __syncthreads();

        // ---- P2: wave wv = value columns 16 wv .. + 15
        const bf16x8_t Vtr[2] = {lds_read_tr_frag(smem, OFF_V, LDW, wv, 0, lane), lds_read_tr_frag(smem, OFF_V, LDW, wv, 1, lane)};
        bf16x8_t bhi[4], blo[4];
#pragma unroll
        for (int s = 0; s < 4; ++s) split_sigma(h[2 * s], h[2 * s + 1], bhi[s], blo[s]);
        // Y[j][v] = ag h + Aak V
        float4_t y[4];
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            float4_t acc = zero4;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const bf16x8_t af = rows_sigma(smem, OFF_AG, LDW, it, s, lane);
                acc = mfma_bf16(af, bhi[s], acc);
                acc = mfma_bf16(af, blo[s], acc);
            }
#pragma unroll
            for (int s = 0; s < 2; ++s) acc = mfma_bf16(rows_sigma(smem, OFF_AAK, LDA, it, s, lane), Vtr[s], acc);
            y[it] = acc;
            __builtin_amdgcn_sched_barrier(0);
        }
        const bf16x8_t Ys[2] = {pack_sigma(y[0], y[1]), pack_sigma(y[2], y[3])};
        if (c + 1 < NT) load_chunk(c + 1, lane, 1);        // the next chunk's inputs travel from here on
        __builtin_amdgcn_sched_barrier(0);
        // SA[i][v] = M Y
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            float4_t acc = zero4;
#pragma unroll
            for (int s = 0; s < 2; ++s) acc = mfma_bf16(lds_read_tr_frag(smem, OFF_MT, LDA, it, s, lane), Ys[s], acc);
            y[it] = acc;
        }
        const bf16x8_t Us[2] = {pack_sigma(y[0], y[1]), pack_sigma(y[2], y[3])};
        if (c + 1 < NT) load_chunk(c + 1, lane, 2);
        __builtin_amdgcn_sched_barrier(0);
        // O[i][v] = qg h + Aqk V + Aqb SA  -> O^T tile [value][token]
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            float4_t acc = zero4;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const bf16x8_t qf = rows_sigma(smem, OFF_QG, LDW, it, s, lane);
                acc = mfma_bf16(qf, bhi[s], acc);
                acc = mfma_bf16(qf, blo[s], acc);
            }
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                acc = mfma_bf16(rows_sigma(smem, OFF_AQK, LDA, it, s, lane), Vtr[s], acc);
                acc = mfma_bf16(rows_sigma(smem, OFF_AQB, LDA, it, s, lane), Us[s], acc);
            }
            store_acc_t(smem, OFF_OT, LDO, wv, it, lane, acc);
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (c + 1 < NT) load_chunk(c + 1, lane, 4);
        // h'[c][v] = e^G h + kg^T V + bg^T SA
        {
            const float* eg = reinterpret_cast<const float*>(smem + OFF_EG);
#pragma unroll
            for (int ct = 0; ct < 8; ++ct) {
                const float4_t e4 = *reinterpret_cast<const float4_t*>(eg + 16 * ct + 4 * g);
                float4_t acc = e4 * h[ct];
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    acc = mfma_bf16(lds_read_tr_frag(smem, OFF_KT, LDW, ct, s, lane), Vtr[s], acc);
                    acc = mfma_bf16(lds_read_tr_frag(smem, OFF_BT, LDW, ct, s, lane), Us[s], acc);
                }
                h[ct] = acc;
                if (ct & 1) __builtin_amdgcn_sched_barrier(0);
            }
        }
        __syncthreads();                   // the O^T tile is complete; every tile of this chunk has been read
        // token 16 tt + x, values 16 wv + 4 g .. + 3: four 8-byte stores per lane
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            const bf16x4_t o4 = lds_read_tr4(smem, OFF_OT, LDO, 16 * wv, tt, lane);
            const int t = c * CH + 16 * tt + x;
            if (t < T) *reinterpret_cast<bf16x4_t*>(o_ + ((sp.tok0 + t) * H + hi) * N + 16 * wv + 4 * g) = o4;
        }
    }
    if (ht != nullptr) {
        const int x = threadIdx.x & 15, g = (threadIdx.x & 63) >> 4;
        float* dst = ht + (int64_t)bh * (N * N) + 16 * wv + x;
#pragma unroll
        for (int ct = 0; ct < 8; ++ct)
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[(16 * ct + 4 * g + e) * N] = h[ct][e];
    }
}

hipError_t launch_fwd_chunk128(const SeqArgs& p, hipStream_t stream) {
    hipError_t e = hipSuccess;
    if (p.cu != nullptr) {             // rows of o behind the last sequence
        e = launch_chunk_items(seq_layout(p, nullptr), nullptr, nullptr, 0, nullptr, tail_of_output(p), stream);
        if (e != hipSuccess) return e;
    }
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(chunk128_fwd_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, LDS128_BYTES);
    if (e != hipSuccess) return e;
    chunk128_fwd_kernel<<<dim3((unsigned)(p.B * p.H)), dim3(512), LDS128_BYTES, stream>>>(
        (const bf16_t*)p.r, (const bf16_t*)p.w, (const bf16_t*)p.k, (const bf16_t*)p.v, (const bf16_t*)p.a,
        (const bf16_t*)p.b, p.h0, p.h0_batch_stride, p.h0_map, p.n_state, (bf16_t*)p.o, p.ht, seq_layout(p, nullptr));
    return hipGetLastError();
}

}  // namespace rwkv7
