// Chunked float32 forward of the RWKV7 generalized delta rule for gfx950: the throughput path for float32
// tensors (K = V = 64), every product on the float32 matrix cores (v_mfma_f32_16x16x4_f32), nothing rounded to
// bf16 anywhere -- the accuracy of the reference's native loop
// (/root/reference/rwkv_ops/rwkv7_kernel/native_keras_op.py:80-88) at several times the speed of walking it
// token by token.
//
// The chunk algebra of the bf16 kernels (the reference's chunk_dplr_fwd,
// /root/reference/rwkv_ops/rwkv7_kernel/torch_op.py:46-120) on chunks of SIXTEEN tokens, the matrix cores'
// smallest tile: with gi / ge the inclusive / exclusive cumulative log decay inside the chunk and G its total,
//     qg = r e^{gi}, ag = a e^{ge}, kt = k e^{-gi}, bt = b e^{-gi}, kg = k e^{G-gi}, bg = b e^{G-gi},
//     Aqk = tril(qg kt^T), Aqb = tril(qg bt^T), Aak = tril_-1(ag kt^T), N = tril_-1(ag bt^T), M = (I - N)^-1,
//     Y = ag h + Aak V,  SA = M Y,  O = qg h + Aqk V + Aqb SA,  h' = diag(e^G) h + kg^T V + bg^T SA.
// One workgroup of four waves per (batch, head) walks the sequence with the state in registers; wave w owns value
// columns 16 w .. + 15.
//
// Register layouts.  For a 16x16 matrix Z write R(Z) for the accumulator layout of the 16x16x4 MFMA: lane (x, g)
// (x = lane % 16, g = lane / 16) holds Z[4 g + e][x], e = 0 .. 3.  One MFMA contracts over four indices, one per
// lane group g; taking for instruction e the indices k = 4 g + e, the four instructions e = 0 .. 3 cover all
// sixteen, and then
//     the B operand of a matrix Z (lane (x, g) supplies Z[k][x]) is R(Z) itself, component e for instruction e,
//     the A operand of a matrix Z (lane (x, g) supplies Z[x][k]) is R(Z^T).
// So an accumulator is the next product's operand as it stands: the state tiles (rows 16 ct + 4 g + e of column x)
// feed ag h and qg h, Y feeds M Y, SA feeds Aqb SA and bg^T SA, and a matrix and its transpose in R layout
// are all the inverse needs:  R(Z1 Z2) = mfma(A = R(Z1^T), B = R(Z2)).
// Operands that come from the inputs lie in LDS as row-major float32 tiles [token][channel]; "row x, four
// consecutive columns" is one 16-byte read and serves four instructions.
#include "rwkv7_f32_mma.h"
#include "rwkv7_kernels.h"
#include "../../include/rwkv7_mi355x.h"

namespace rwkv7 {

namespace {

constexpr int LDC = 20;                        // row stride (floats) of the transposed tiles [64 channels][16 tokens]
constexpr int TILE_C = NH * LDC * 4;           // bytes of a transposed one (large enough to hold a row-major tile too)
static_assert(TILE_C >= TILE_F, "the strong-decay path keeps a row-major tile in a transposed tile's place");
// one buffer = everything the consumer waves need of one chunk; three buffers, chunk c in buffer c % 3
constexpr int F_QG = 0, F_AG = TILE_F, F_KT = 2 * TILE_F, F_BT = 3 * TILE_F;        // row-major
constexpr int F_KGT = 4 * TILE_F, F_BGT = F_KGT + TILE_C, F_VT = F_BGT + TILE_C;    // transposed: kg^T, bg^T, V^T
constexpr int F_BOX = F_VT + TILE_C;           // four 1 KiB mailboxes, one float4 per lane: R(Aqk^T), R(Aqb^T), R(Aak^T), R(M^T)
constexpr int F_EG = F_BOX + 4 * 1024;         // float [64]: e^G per key channel
constexpr int F_FLAG = F_EG + 256;             // int [4]: per-producer-wave "strong decay" flags
constexpr int F_SCR = F_FLAG + 64;             // 1 KiB: the wave that inverts transposes N through here
constexpr int BUF_BYTES = F_SCR + 1024;
constexpr int F_DEC = F_QG, F_RAW_R = F_KGT;   // strong chunks: per-step decays and raw r (row-major) in these places
constexpr int LDS_F32_BYTES = 3 * BUF_BYTES;
static_assert(LDS_F32_BYTES <= 160 * 1024, "one workgroup per CU");

}  // namespace

// Twelve waves in three roles, one barrier per round.  In round r
//   * waves 0-3, the consumers, apply chunk r - 2 to the state (all matrix instructions),
//   * one group of four producer waves turns chunk r - 1's operand tiles into the three intra-chunk matrices and M,
//   * the other group turns chunk r's inputs into operand tiles (vector arithmetic),
// none of which depends on the state.  Waves 4-7 take the even chunks, waves 8-11 the odd ones: a group spends two
// rounds on a chunk, so the request for its next chunk's inputs, issued when the tiles are written, has two rounds
// to arrive.  Three buffers of tiles, chunk c in buffer c % 3.
// WITH_O = false: the pass that only leaves the states for the backward (o_ is NULL): the three products of O, the
// two matrices and the tile they need are left out.
template <bool WITH_O>
__global__ __launch_bounds__(768)
void chunk16_f32_fwd_kernel(const float* __restrict__ r_, const float* __restrict__ w_, const float* __restrict__ k_,
                            const float* __restrict__ v_, const float* __restrict__ a_, const float* __restrict__ b_,
                            const float* __restrict__ h0, int64_t h0_batch_stride, const int* __restrict__ h0_map,
                            int n_state, float* __restrict__ o_, float* __restrict__ ht, SeqLayout L,
                            float* __restrict__ seg_states, int seg, int* __restrict__ strong_out)
{
    // seg_states: the state BEFORE token t is stored for every t that is a multiple of `seg` (a multiple of 16),
    // dense batches [workgroup][t / seg][64][64], packed sequences (seg = 16 only) the records of f32_chunk_records: what the
    // backward kernels restart from.  o_ may then be NULL.
    // strong_out (nullable): one integer per workgroup, 1 when a chunk of its sequence was walked token by token.
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_all[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int w = wave & 3;                    // consumers: value columns 16 w .. + 15; producers: channels 16 w .. + 15
    const bool producer = wave >= 4;
    const int H = L.H;
    const int bh = blockIdx.x, hi = bh % H, bi = bh / H;
    const SeqSpan sp = seq_span(L, bi);
    const int T = sp.len, NT = (T + C16 - 1) / C16;
    const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
    if (NT == 0) {                             // a sequence without tokens: the state passes through
        if (strong_out != nullptr && threadIdx.x == 0) strong_out[bh] = 0;
        if (!producer && ht != nullptr) {
            const int x = threadIdx.x & 15, g = (threadIdx.x & 63) >> 4;
            float* dst = ht + (int64_t)bh * (NH * NH) + 16 * w + x;
            const float* src = h0 == nullptr ? nullptr
                : h0 + state_row(h0_map, n_state, bi) * h0_batch_stride + (int64_t)hi * (NH * NH) + 16 * w + x;
            for (int i = 0; i < 16; ++i) dst[(4 * i + g) * NH] = src ? src[(4 * i + g) * NH] : 0.f;
        }
        return;
    }
    const int ROUNDS = NT + 2;                 // every wave passes exactly this many barriers

    if (producer) {
        // ================================================================== producers
        const int parity = (wave >> 2) - 1;    // this group's chunks: parity, parity + 2, ...
        // The inputs of a chunk in the load layout: lane (x, g) holds channels 16 w + 4 g .. + 3 of token x.
        struct Inputs { float4_t R4, W4, K4, V4, A4, B4; };
        auto load_chunk = [&](Inputs& in, int c, int ln) {
            const int t = c * C16 + (ln & 15);
            // rows past the sequence's end are read from the last valid row and zeroed by the consumer of the registers
            const int64_t row = ((sp.tok0 + (t < T ? t : T - 1)) * H + hi) * NH + 16 * w + 4 * (ln >> 4);
            in.W4 = *reinterpret_cast<const float4_t*>(w_ + row); in.R4 = *reinterpret_cast<const float4_t*>(r_ + row);
            in.K4 = *reinterpret_cast<const float4_t*>(k_ + row); in.V4 = *reinterpret_cast<const float4_t*>(v_ + row);
            in.A4 = *reinterpret_cast<const float4_t*>(a_ + row); in.B4 = *reinterpret_cast<const float4_t*>(b_ + row);
        };
        Inputs next;                           // the group's next chunk, on its way
        load_chunk(next, parity, (int)(threadIdx.x & 63));       // (past the end: the last token again, never used)
        for (int i = 0; i < parity; ++i) __syncthreads();
        int passed = parity;
        for (int c = parity; c < NT; c += 2) {
            int lane = threadIdx.x & 63;
            asm volatile("" : "+v"(lane));     // (per-lane addresses are formed where they are used, not kept across rounds)
            const int x = lane & 15, g = lane >> 4;
            unsigned char* smem = smem_all + (c % 3) * BUF_BYTES;
            const int ch = 16 * w + 4 * g;
            const bool valid = c * C16 + x < T;
            auto put4 = [&](int off, float4_t val) {
                *reinterpret_cast<float4_t*>(smem + off + (x * LDF + ch) * 4) = val;
            };
            auto put4t = [&](int off, float4_t val) {              // transposed tile: [channel][token]
#pragma unroll
                for (int e = 0; e < 4; ++e) *reinterpret_cast<float*>(smem + off + ((ch + e) * LDC + x) * 4) = val[e];
            };
            // ---------------------------------------------------------------- round c: the operand tiles
            Inputs cur = next;
            load_chunk(next, c + 2, lane);     // two rounds ahead
            if (!valid) { cur.R4 = cur.K4 = cur.V4 = cur.A4 = cur.B4 = zero4; }
            float4_t gstep;
            {
                // cumulative log decays (base 2) over the chunk's tokens = the lanes of a DPP row
                float4_t gi, G;
                const float vmask = valid ? 1.f : 0.f;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    gstep[e] = vmask * fmaxf(-LOG2E * ex2(LOG2E * cur.W4[e]), G_MIN2);   // log2 of exp(-exp(w))
                    gi[e] = row_inclusive_scan(gstep[e]);
                    G[e] = row_sum(gstep[e]);
                }
                const bool strong_here = fminf(fminf(G[0], G[1]), fminf(G[2], G[3])) < -STRONG2;
                const bool strong_wave = __builtin_amdgcn_ballot_w64(strong_here) != 0ull;
                if (lane == 0) reinterpret_cast<int*>(smem + F_FLAG)[w] = strong_wave ? 1 : 0;
                if (x == 0)
                    *reinterpret_cast<float4_t*>(smem + F_EG + ch * 4) = float4_t{ex2(G[0]), ex2(G[1]), ex2(G[2]), ex2(G[3])};
                float4_t qg, ag, kt, bt, kg, bg;                   // (in a strong chunk these may overflow; nobody reads them)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float up = ex2(-gi[e]), tail = ex2(G[e] - gi[e]);
                    qg[e] = cur.R4[e] * ex2(gi[e]);
                    ag[e] = cur.A4[e] * ex2(gi[e] - gstep[e]);
                    kt[e] = cur.K4[e] * up;  bt[e] = cur.B4[e] * up;
                    kg[e] = cur.K4[e] * tail; bg[e] = cur.B4[e] * tail;
                }
                put4(F_QG, qg); put4(F_AG, ag); put4(F_KT, kt); put4(F_BT, bt);
                put4t(F_KGT, kg); put4t(F_BGT, bg);
                put4t(F_VT, cur.V4);
            }
            __syncthreads();
            // ---------------------------------------------------------------- round c + 1: the matrices
            bool strong;
            {
                const int* fl = reinterpret_cast<const int*>(smem + F_FLAG);
                strong = (fl[0] | fl[1] | fl[2] | fl[3]) != 0;
            }
            if (strong) {
                // Strong decays (never with RWKV7's own parameterisation): the consumers will walk this chunk token by
                // token; the per-step decays and the raw inputs take the place of the scaled operands.
                float4_t dec;
#pragma unroll
                for (int e = 0; e < 4; ++e) dec[e] = ex2(gstep[e]);             // rows past the end: 1
                put4(F_DEC, dec); put4(F_AG, cur.A4); put4(F_KT, cur.K4); put4(F_BT, cur.B4); put4(F_RAW_R, cur.R4);
            } else {
                // The intra-chunk matrices, each as R of its transpose: lane (x = i, g) holds A[i][4 g + e].
                // D[j][i] = sum_c X[j][c] Y[i][c]: both operands are "row x, four consecutive channels" of a tile.
                auto gram = [&](int off_rows_j, int off_rows_i) {
                    float4_t acc = zero4;
#pragma unroll
                    for (int ct = 0; ct < 4; ++ct) {
                        const float4_t aj = tile4(smem, off_rows_j, x, 16 * ct + 4 * g);
                        const float4_t bi4 = tile4(smem, off_rows_i, x, 16 * ct + 4 * g);
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc = mfma_f32(aj[e], bi4[e], acc);
                    }
                    return acc;
                };
                if (w != 2) {
                  if (WITH_O || w == 1) {
                    // producers 0, 1, 3: Aqk, Aak, Aqb
                    float4_t acc = gram(w == 3 ? F_BT : F_KT, w == 1 ? F_AG : F_QG);  // rows j = 4 g + e, column i = x
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int j = 4 * g + e;
                        if (w == 1 ? j >= x : j > x) acc[e] = 0.f;                      // j < i (Aak), j <= i (Aqk, Aqb)
                    }
                    const int box = w == 0 ? 0 : (w == 3 ? 1 : 2);
                    *reinterpret_cast<float4_t*>(smem + F_BOX + box * 1024 + lane * 16) = acc;
                  }
                } else {
                    // producer 2: N = tril_-1(ag bt^T) and M = (I - N)^-1 = (I + N)(I + N^2)(I + N^4)(I + N^8)
                    float4_t NT_ = gram(F_BT, F_AG);   // R(N^T): lane (x = i, g): N[i][4 g + e]
#pragma unroll
                    for (int e = 0; e < 4; ++e) if (4 * g + e >= x) NT_[e] = 0.f;      // keep j < i
                    // R(N): lane (x = j, g): N[4 g + e][j] -- the transpose, through this wave's own kilobyte of LDS
                    float4_t Nm;
                    {
                        float* scr = reinterpret_cast<float*>(smem + F_SCR);
                        *reinterpret_cast<float4_t*>(scr + x * 16 + 4 * g) = NT_;      // N[i = x][4 g ..] row-major
#pragma unroll
                        for (int e = 0; e < 4; ++e) Nm[e] = scr[(4 * g + e) * 16 + x];
                    }
                    // Only R(M^T) is needed (the A operand of M Y).  With D the product so far and P the current power:
                    // R(D^T) += R(P^T D^T) = mfma(A = R(P), B = R(D^T)).
                    float4_t MT = NT_;
#pragma unroll
                    for (int e = 0; e < 4; ++e) if (4 * g + e == x) MT[e] += 1.f;
                    float4_t P = Nm, PT = NT_;
#pragma unroll
                    for (int it = 0; it < 3; ++it) {
                        float4_t P2 = zero4, P2T = zero4;
#pragma unroll
                        for (int e = 0; e < 4; ++e) P2 = mfma_f32(PT[e], P[e], P2);       // R(P P)
                        if (it < 2) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) P2T = mfma_f32(P[e], PT[e], P2T); // R(P^T P^T)
                        }
                        P = P2; PT = P2T;
                        float4_t upd = MT;
#pragma unroll
                        for (int e = 0; e < 4; ++e) upd = mfma_f32(P[e], MT[e], upd);     // R(D^T) + R(P^T D^T)
                        MT = upd;
                    }
                    *reinterpret_cast<float4_t*>(smem + F_BOX + 3 * 1024 + lane * 16) = MT;
                }
            }
            __syncthreads();
            passed += 2;
        }
        for (; passed < ROUNDS; ++passed) __syncthreads();
        return;
    }

    // ====================================================================== consumers
    // state: tile ct = rows 16 ct + 4 g + e of column 16 w + x
    float4_t h[4];
    {
        const int x = threadIdx.x & 15, g = (threadIdx.x & 63) >> 4;
        if (h0 != nullptr) {
            const float* src = h0 + state_row(h0_map, n_state, bi) * h0_batch_stride + (int64_t)hi * (NH * NH) + 16 * w + x;
#pragma unroll
            for (int ct = 0; ct < 4; ++ct)
#pragma unroll
                for (int e = 0; e < 4; ++e) h[ct][e] = src[(16 * ct + 4 * g + e) * NH];
        } else {
#pragma unroll
            for (int ct = 0; ct < 4; ++ct) h[ct] = zero4;
        }
    }
    __syncthreads();                           // rounds 0 and 1: the first chunk is on its way
    __syncthreads();
    // where the states go: dense [workgroup][t / seg], packed the records of the float32 backward (seg = 16)
    const ChunkRecords packed_recs = f32_chunk_records(L, sp, bi, hi, NT);
    const int64_t seg_first = L.cu != nullptr ? packed_recs.first : (int64_t)bh * ((T + seg - 1) / seg);
    const int seg_step = L.cu != nullptr ? packed_recs.step : 1;
    bool any_strong = false;
    for (int c = 0; c < NT; ++c) {             // round c + 2
        int lane = threadIdx.x & 63;
        asm volatile("" : "+v"(lane));
        const int x = lane & 15, g = lane >> 4;
        const unsigned char* smem = smem_all + (c % 3) * BUF_BYTES;
        const bool valid = c * C16 + x < T;
        if (seg_states != nullptr && (c * C16) % seg == 0) {
            float* dst = seg_states + (seg_first + (int64_t)((c * C16) / seg) * seg_step) * (NH * NH) + 16 * w + x;
#pragma unroll
            for (int ct = 0; ct < 4; ++ct)
#pragma unroll
                for (int e = 0; e < 4; ++e) dst[(16 * ct + 4 * g + e) * NH] = h[ct][e];
        }
        bool strong;
        {
            const int* fl = reinterpret_cast<const int*>(smem + F_FLAG);
            strong = (fl[0] | fl[1] | fl[2] | fl[3]) != 0;
        }
        any_strong |= strong;
        if (strong) {
            // token by token in float32 on the state as it lies in the registers
            const int nt = T - c * C16 < C16 ? T - c * C16 : C16;
            for (int tt = 0; tt < nt; ++tt) {
                const float vv = *reinterpret_cast<const float*>(smem + F_VT + ((16 * w + x) * LDC + tt) * 4);
                float4_t sa4 = zero4;
#pragma unroll
                for (int ct = 0; ct < 4; ++ct) sa4 += tile4(smem, F_AG, tt, 16 * ct + 4 * g) * h[ct];
                float sa = (sa4[0] + sa4[1]) + (sa4[2] + sa4[3]);
                sa = sum_over_rows(sa);
                float4_t o4 = zero4;
#pragma unroll
                for (int ct = 0; ct < 4; ++ct) {
                    const int col = 16 * ct + 4 * g;
                    h[ct] = tile4(smem, F_DEC, tt, col) * h[ct] + tile4(smem, F_BT, tt, col) * sa + tile4(smem, F_KT, tt, col) * vv;
                    o4 += tile4(smem, F_RAW_R, tt, col) * h[ct];
                }
                float ov = (o4[0] + o4[1]) + (o4[2] + o4[3]);
                ov = sum_over_rows(ov);
                if (g == 0 && o_ != nullptr) o_[((sp.tok0 + c * C16 + tt) * H + hi) * NH + 16 * w + x] = ov;
            }
            __syncthreads();
            continue;
        }
        const float4_t AqkT = *reinterpret_cast<const float4_t*>(smem + F_BOX + 0 * 1024 + lane * 16);
        const float4_t AqbT = *reinterpret_cast<const float4_t*>(smem + F_BOX + 1 * 1024 + lane * 16);
        const float4_t AakT = *reinterpret_cast<const float4_t*>(smem + F_BOX + 2 * 1024 + lane * 16);
        const float4_t MT = *reinterpret_cast<const float4_t*>(smem + F_BOX + 3 * 1024 + lane * 16);
        // Vg[e] = V[token 4 g + e][16 w + x]: R of V restricted to this wave's columns
        const float4_t Vg = *reinterpret_cast<const float4_t*>(smem + F_VT + ((16 * w + x) * LDC + 4 * g) * 4);
        // R(Y): Y[j][v] = ag h + Aak V, and the part of O that does not need SA, two independent chains of matrix
        // instructions issued alternately (an instruction that accumulates onto the previous one's result waits for it).
        // R(O^T): O^T[v][i] = h^T qg^T + V^T Aqk^T + SA^T Aqb^T -- the operands of O with A and B exchanged, so that
        // a lane ends up with four consecutive values of ONE token and stores them as 16 bytes
        float4_t Y = zero4, OT = zero4;
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
            const float4_t af = tile4(smem, F_AG, x, 16 * ct + 4 * g);
            const float4_t qf = tile4(smem, F_QG, x, 16 * ct + 4 * g);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                Y = mfma_f32(af[e], h[ct][e], Y);
                if constexpr (WITH_O) OT = mfma_f32(h[ct][e], qf[e], OT);
            }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            Y = mfma_f32(AakT[e], Vg[e], Y);
            if constexpr (WITH_O) OT = mfma_f32(Vg[e], AqkT[e], OT);
        }
        // R(SA): SA = M Y
        float4_t SA = zero4;
#pragma unroll
        for (int e = 0; e < 4; ++e) SA = mfma_f32(MT[e], Y[e], SA);
        // h'[c][v] = e^G h + kg^T V + bg^T SA: the A operand is kg[token 4 g + e][channel 16 ct + x], a row of kg^T
        // (the four tiles and the last of O are five independent chains: one instruction of each in turn; the part
        // that does not need SA first)
        {
            const float* eg = reinterpret_cast<const float*>(smem + F_EG);
            float4_t kgf[4], bgf[4];
#pragma unroll
            for (int ct = 0; ct < 4; ++ct) {
                h[ct] = *reinterpret_cast<const float4_t*>(eg + 16 * ct + 4 * g) * h[ct];
                kgf[ct] = *reinterpret_cast<const float4_t*>(smem + F_KGT + ((16 * ct + x) * LDC + 4 * g) * 4);
                bgf[ct] = *reinterpret_cast<const float4_t*>(smem + F_BGT + ((16 * ct + x) * LDC + 4 * g) * 4);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int ct = 0; ct < 4; ++ct) h[ct] = mfma_f32(kgf[ct][e], Vg[e], h[ct]);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if constexpr (WITH_O) OT = mfma_f32(SA[e], AqbT[e], OT);
#pragma unroll
                for (int ct = 0; ct < 4; ++ct) h[ct] = mfma_f32(bgf[ct][e], SA[e], h[ct]);
            }
        }
        if (WITH_O && valid && o_ != nullptr)
            *reinterpret_cast<float4_t*>(o_ + ((sp.tok0 + c * C16 + x) * H + hi) * NH + 16 * w + 4 * g) = OT;
        __syncthreads();
    }
    if (strong_out != nullptr && threadIdx.x == 0) strong_out[bh] = any_strong ? 1 : 0;
    if (ht != nullptr) {
        const int x = threadIdx.x & 15, g = (threadIdx.x & 63) >> 4;
        float* dst = ht + (int64_t)bh * (NH * NH) + 16 * w + x;
#pragma unroll
        for (int ct = 0; ct < 4; ++ct)
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[(16 * ct + 4 * g + e) * NH] = h[ct][e];
    }
}

hipError_t launch_fwd_chunk_f32(const SeqArgs& p, hipStream_t stream) {
    if (p.cu != nullptr) {             // rows of o behind the last sequence
        hipError_t e0 = launch_chunk_items(seq_layout(p, nullptr), nullptr, nullptr, 0, nullptr, tail_of_output(p), stream);
        if (e0 != hipSuccess) return e0;
    }
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(chunk16_f32_fwd_kernel<true>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, LDS_F32_BYTES);
    if (e != hipSuccess) return e;
    chunk16_f32_fwd_kernel<true><<<dim3((unsigned)(p.B * p.H)), dim3(768), LDS_F32_BYTES, stream>>>(
        (const float*)p.r, (const float*)p.w, (const float*)p.k, (const float*)p.v, (const float*)p.a,
        (const float*)p.b, p.h0, p.h0_batch_stride, p.h0_map, p.n_state, (float*)p.o, p.ht, seq_layout(p, nullptr),
        nullptr, 0, nullptr);
    return hipGetLastError();
}

// the forward without outputs, storing the state at the start of every segment of `seg` tokens (float32 tensors,
// K = V = 64; seg a multiple of 16, dense batches, or 16 with packed sequences (p.cu)); strong (nullable): per
// (batch, head) whether a chunk's decay was too strong for the chunk form
hipError_t launch_fwd_chunk_f32_states(const SeqArgs& p, float* states, int seg, hipStream_t stream, int* strong) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(chunk16_f32_fwd_kernel<false>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, LDS_F32_BYTES);
    if (e != hipSuccess) return e;
    chunk16_f32_fwd_kernel<false><<<dim3((unsigned)(p.B * p.H)), dim3(768), LDS_F32_BYTES, stream>>>(
        (const float*)p.r, (const float*)p.w, (const float*)p.k, (const float*)p.v, (const float*)p.a,
        (const float*)p.b, p.h0, p.h0_batch_stride, nullptr, 0, nullptr, nullptr, seq_layout(p, nullptr), states, seg,
        strong);
    static_assert(C16 == 16, "packed records are per 16-token chunk");
    return hipGetLastError();
}

}  // namespace rwkv7
