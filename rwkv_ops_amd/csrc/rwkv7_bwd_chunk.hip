// Chunked backward of the RWKV7 generalized delta rule for gfx950 (bf16 inputs).
//
// What the reference does in twelve Triton launches
// (/root/reference/rwkv_ops/rwkv7_kernel/torch_op.py:123-265: five forward recomputations, then
// dAu, the reverse state scan dhu, dv, bwd_o, bwd_wy, dqk_intra and dgk) is done in four kernels:
//
//   1. chunk_summary_kernel<MODE_BWD> (rwkv7_fwd_chunk.hip) per chunk: Pp, Qc, eG of the chunk's affine
//      action  O = Qt h0 + OI,  h' = (diag(eG) + Pp) h0 + Qc,  and the product Qt^T dO.
//   2. chunk_scans_kernel, two serial scans in one launch: the state scan stores the state h0 at the
//      start of every chunk; the reverse scan (last chunk first) is the adjoint of that affine action,
//      dh0 = (diag(eG) + Pp^T) dh' + Qt^T dO   (chunk_h_bwd.py:27-157 does the same with w, qg, bg
//      unfolded), stores dh' for every chunk and returns the gradient of the initial state.
//   3. chunk_bwd_kernel             per chunk, fully parallel: recomputes the chunk's forward
//      quantities from the inputs and h0, and back-propagates through them.
//   4. chunk_bwd_general_kernel     the same for the chunks whose decay needs several exponent buckets.
//
// Per chunk, with gi/ge the inclusive/exclusive cumulative log decay, G its total, and
//   qg = r e^{gi}, ag = a e^{ge}, kt = k e^{-gi}, bt = b e^{-gi}, kg = k e^{G-gi}, bg = b e^{G-gi},
//   Aqk = tril(qg kt^T), Aqb = tril(qg bt^T), Aak = tril_-1(ag kt^T), Aab = tril_-1(ag bt^T),
//   M = (I - Aab)^-1,  Y = ag h0 + Aak V,  SA = M Y,
//   O = qg h0 + Aqk V + Aqb SA,   h' = diag(e^G) h0 + kg^T V + bg^T SA :
//   dSA = Aqb^T dO + bg dh'            dY = M^T dSA
//   dV  = Aqk^T dO + kg dh' + Aak^T dY
//   dAqk = tril(dO V^T)  dAqb = tril(dO SA^T)  dAak = tril_-1(dY V^T)  dAab = tril_-1(dY SA^T)
//   dqg = dO h0^T + dAqk kt + dAqb bt      dag = dY h0^T + dAak kt + dAab bt
//   dkt = dAqk^T qg + dAak^T ag            dbt = dAqb^T qg + dAab^T ag
//   dkg = V dh'^T                          dbg = SA dh'^T
//   dr = dqg e^{gi}   da = dag e^{ge}   dk = dkt e^{-gi} + dkg e^{G-gi}   db = dbt e^{-gi} + dbg e^{G-gi}
//   dgi = dr r - dk k - db b,  dge = da a,  dG = e^G sum_v(h0 dh') + sum_t (dkg e^{G-gi} k + dbg e^{G-gi} b)
//   dg_t = sum_{s >= t}(dgi_s + dge_s) - dge_t + dG,   dw = dg g          (g = -exp(w))
// (the reference's formulas: chunk_o_bwd.py:27-139,152-294,309-382, wy_fast_bwd.py:142-192,
//  chunk_A_bwd.py:21-328; here the triangular inverse is differentiated through SA = M Y directly,
//  which gives dAab = dY SA^T without forming dM).
//
// chunk_bwd_kernel is written as tile algebra: every operand is a row-major 64x64 bf16 tile in LDS
// that is read either along its rows (16-byte reads) or along its columns (ds_read_b64_tr_b16), so
// any product of two tiles or their transposes is one call; every product's accumulators (column
// fixed per lane, four consecutive rows) are stored transposed with 8-byte writes.  The decay
// buckets of the forward kernel carry over: each bucket is one pass of the last group of products
// with its own exponent offset.
#include <type_traits>
#include "rwkv7_chunk.h"
#include "rwkv7_kernels.h"
#include "../../include/rwkv7_mi355x.h"

namespace rwkv7 {

namespace {

// Log decays are kept in base 2 (as in rwkv7_fwd_chunk.hip), so every exponential is one v_exp_f32.
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;
constexpr float BUCKET2 = BUCKET * LOG2E;      // exponent range of one decay bucket, in base-2 units
constexpr float G_MIN2 = G_MIN * LOG2E;        // per-step log-decay clamp, in base-2 units
__device__ __forceinline__ float ex2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ bf16x8_t join4(bf16x4_t lo, bf16x4_t hi) {
    bf16x8_t r = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return r;
}

// ------------------------------------------------------------------------------------------------
// K2 / K3: the two serial scans, one code.  Both are  x <- diag(eG) x + A x + C  per chunk with x a
// 64x64 float32 image held in MFMA accumulators (wave = 16 value columns):
//   K2 (REVERSE = false): h, first chunk first, A = Pp ([4 tiles][2 k-steps][2 halves][64][4]), C = Qc;
//      stores h at the START of every chunk:  hs[n][4 value tiles][4 key tiles][64 lanes][4];
//   K3 (REVERSE = true):  dh, last chunk first, A = Pp^T (read out of the same Pp fragments), C = Qt^T dO
//      (chunk_h_bwd.py:27-157 does the same with w, qg, bg unfolded); stores dh at the END of every
//      chunk in the same image layout, and finally the gradient of the initial state.
// The chain is serial, so four chunks' operands are kept in flight: register sets requested four
// chunks ahead, copied through a double-buffered LDS stage and read from there as fragments.
constexpr int SCAN2_STAGE_BYTES = 2 * 8192 + 256;          // A | C | eG

template <bool REVERSE>
__device__ __forceinline__
void chunk_affine_scan(unsigned char* smem, int bh, const bf16_t* __restrict__ A_, const bf16_t* __restrict__ C_,
                       const float* __restrict__ eg, const float* __restrict__ x0, int64_t x0_batch_stride,
                       float* __restrict__ xs, float* __restrict__ x_final, const SeqLayout& L)
{
    const int tid = threadIdx.x;
    const int lane = tid & 63, vt = tid >> 6;
    const int x = lane & 15, g = lane >> 4;
    const int hi = bh % L.H, bi = bh / L.H;
    const SeqSpan sp = seq_span(L, bi);
    const int NT = (sp.len + CH - 1) / CH;
    float4_t h[4];
    if (x0 != nullptr) {
        const float* src = x0 + (int64_t)bi * x0_batch_stride + (int64_t)hi * STATE + 16 * vt + x;
#pragma unroll
        for (int ct = 0; ct < 4; ++ct)
#pragma unroll
            for (int e = 0; e < 4; ++e) h[ct][e] = src[(16 * ct + 4 * g + e) * HEAD];
    } else {
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) h[ct] = float4_t{0.f, 0.f, 0.f, 0.f};
    }
    struct Set { float4_t q[4]; float4_t e; };
    auto chunk_of = [&](int i) { return REVERSE ? NT - 1 - i : i; };
    auto request = [&](int i, Set& S) {                 // i-th chunk of the walk, 16-byte piece j * 256 + tid
        if (i >= NT) return;
        const int64_t n = chunk_record(L, sp, bi, hi, chunk_of(i));
#pragma unroll
        for (int j = 0; j < 4; ++j)
            S.q[j] = *reinterpret_cast<const float4_t*>((j < 2 ? A_ : C_) + n * 4096 + ((j & 1) * 256 + tid) * 8);
        if (tid < 16) S.e = *reinterpret_cast<const float4_t*>(eg + n * HEAD + 4 * tid);
    };
    auto step = [&](int i, Set& S) {
        if (i >= NT) return;
        unsigned char* st = smem + (i & 1) * SCAN2_STAGE_BYTES;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            *reinterpret_cast<float4_t*>(st + (j >> 1) * 8192 + ((j & 1) * 256 + tid) * 16) = S.q[j];
        if (tid < 16) *reinterpret_cast<float4_t*>(st + 2 * 8192 + tid * 16) = S.e;
        request(i + 4, S);                              // this set's next turn
        const int64_t n = chunk_record(L, sp, bi, hi, chunk_of(i));
#pragma unroll
        for (int ct = 0; ct < 4; ++ct)
            *reinterpret_cast<float4_t*>(xs + n * 4096 + ((vt * 4 + ct) * 64 + lane) * 4) = h[ct];
        bf16x8_t bhi[2], blo[2];
        split_sigma(h[0], h[1], bhi[0], blo[0]);
        split_sigma(h[2], h[3], bhi[1], blo[1]);
        __syncthreads();
        const bf16_t* fa = reinterpret_cast<const bf16_t*>(st);
        const bf16x4_t* fc = reinterpret_cast<const bf16x4_t*>(st + 8192);
        const float* fe = reinterpret_cast<const float*>(st + 2 * 8192);
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
            const float4_t e4 = *reinterpret_cast<const float4_t*>(fe + 16 * ct + 4 * g);
            float4_t acc = unpack4(fc[(vt * 4 + ct) * 64 + lane]) + e4 * h[ct];
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                bf16x8_t a8;
                if constexpr (REVERSE) {
                    // A = Pp^T, read out of Pp's own fragments: slot (h', e') of lane (x', g') is
                    // Pp[32 s + 16 h' + 4 g' + e'][16 ct + x'], which lies in fragment (tile 2 s + h', piece ct)
                    // at lane 16 (x' / 4) + 4 g' + e', element x' % 4 - exactly what the transposing read
                    // delivers when source lane p of a 16-lane group points at lane 16 (p % 4) + 4 g' + p / 4.
                    const int p16 = lane & 15;
                    const int src = 16 * (p16 & 3) + 4 * g + (p16 >> 2);
                    const bf16_t* q0 = fa + (((2 * s) * 4 + ct) * 64 + src) * 4;
                    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((RWKV7_LDS s16x4_t*)(q0));
                    const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((RWKV7_LDS s16x4_t*)(q0 + 4 * 64 * 4));
                    typedef short s16x8_t __attribute__((ext_vector_type(8)));
                    const s16x8_t r8 = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
                    a8 = __builtin_bit_cast(bf16x8_t, r8);
                } else
                    a8 = join4(*reinterpret_cast<const bf16x4_t*>(fa + ((ct * 4 + 2 * s) * 64 + lane) * 4),
                               *reinterpret_cast<const bf16x4_t*>(fa + ((ct * 4 + 2 * s + 1) * 64 + lane) * 4));
                acc = mfma_bf16(a8, bhi[s], acc);
                acc = mfma_bf16(a8, blo[s], acc);
            }
            h[ct] = acc;                                // all four tiles read the OLD x through bhi/blo
        }
    };
    Set S0, S1, S2, S3;
    request(0, S0); request(1, S1); request(2, S2); request(3, S3);
    for (int i = 0; i < NT; i += 4) {
        step(i, S0); step(i + 1, S1); step(i + 2, S2); step(i + 3, S3);
    }
    if (x_final != nullptr) {
        float* dst = x_final + (int64_t)bh * STATE + 16 * vt + x;
#pragma unroll
        for (int ct = 0; ct < 4; ++ct)
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[(16 * ct + 4 * g + e) * HEAD] = h[ct][e];
    }
}

// K2 and K3 do not depend on each other and each fills only B*H workgroups, so they share a launch:
// workgroups [0, BH) run the state scan, [BH, 2 BH) the adjoint scan.
__global__ __launch_bounds__(256)
void chunk_scans_kernel(const bf16_t* __restrict__ pp, const bf16_t* __restrict__ qc,
                        const bf16_t* __restrict__ qdo,
                        const float* __restrict__ eg, const float* __restrict__ h0, int64_t h0_batch_stride,
                        const float* __restrict__ dht, float* __restrict__ hs, float* __restrict__ dhs,
                        float* __restrict__ dh0, SeqLayout L, unsigned* __restrict__ list)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    // also clears the count of the multi-bucket chunk list that chunk_bwd_kernel fills later
    if (blockIdx.x == 0 && threadIdx.x == 0) list[0] = 0u;
    const int BH = gridDim.x >> 1;
    if ((int)blockIdx.x < BH)
        chunk_affine_scan<false>(smem, (int)blockIdx.x, pp, qc, eg, h0, h0_batch_stride, hs, nullptr, L);
    else
        chunk_affine_scan<true>(smem, (int)blockIdx.x - BH, pp, qdo, eg, dht, (int64_t)L.H * STATE, dhs, dh0, L);
}

// ------------------------------------------------------------------------------------------------
// K4.  LDS: 15 tile slots of 10 KiB and a small scratch area.
constexpr int SLOT(int i) { return i * TILE_BYTES; }
constexpr int S_QG = SLOT(0), S_AG = SLOT(1), S_KT = SLOT(2), S_BT = SLOT(3), S_V = SLOT(4), S_DO = SLOT(5);
constexpr int S_AQK = SLOT(6), S_AQB = SLOT(7), S_AAK = SLOT(8);
constexpr int S_AAB = SLOT(9), S_H0 = SLOT(9), S_DAQK = SLOT(9);          // Aab -> h0^T -> dAqk
constexpr int S_MT = SLOT(10), S_DAQB = SLOT(10);                          // M^T -> dAqb
constexpr int S_Y = SLOT(11), S_DH = SLOT(11), S_DY = SLOT(11);            // Y^T -> dh'^T -> dY^T
constexpr int S_SA = SLOT(12);                                             // SA^T
constexpr int S_BG = SLOT(13), S_KG = SLOT(13), S_DAAK = SLOT(13);         // bg -> kg -> dAak
constexpr int S_DSA = SLOT(14), S_DAAB = SLOT(14);                         // dSA^T -> dAab
constexpr int S_STAGE0 = SLOT(4), S_STAGE1 = SLOT(6), S_STAGE2 = SLOT(11); // float staging, 2 slots each
// The one-bucket kernel has no bg / kg tile, which leaves two slots free from the start: h0^T and dh'^T get slots of
// their own and are written in the prologue, and every later tile lands in a slot whose previous tenant's last read
// lies behind a barrier that is needed anyway.  Its plan where it differs from the one above:
//   9: Aab -> dSA^T -> dAqk    7: Aqb -> dAak    13: h0^T    14: dh'^T -> dAab    11: Y^T -> dY^T
constexpr int S1_H0 = SLOT(13), S1_DH = SLOT(14), S1_DSA = SLOT(9), S1_DAAK = SLOT(7);
constexpr int OFF_TOT = SLOT(15);            // float [4][64]  sub-block totals of the log decay
constexpr int OFF_DI = OFF_TOT + 1024;       // 4 inverted diagonal blocks, bf16 16x16
constexpr int OFF_RED = OFF_DI + 2048;       // float [4][64] + [4][64] reduction scratch
constexpr int OFF_EGB = OFF_RED + 2048;      // float [64]: decay of the whole chunk per key channel
constexpr int BWD_LDS_BYTES = OFF_EGB + 256;
constexpr int LDZ = 68;                      // row stride (floats) of a staging tile [channel][token]

// Eight waves: wave (w, hf) = (id & 3, id >> 2).  In the load layout (prologue and epilogue) a lane owns
// token 16w + x and the eight channels 32hf + 8g .. +7; in the tile algebra a wave owns the 16 output
// columns of column tile w and the two row tiles 2hf, 2hf + 1.  Two waves per SIMD hide each other's
// LDS and MFMA latencies, and every per-lane array is half as long as it would be with four waves.
//
// The global inputs of one chunk in the load layout, as one lane holds them.  chunk_bwd_kernel requests
// those of its next chunk while it finishes the current one.
struct ChunkInputs {
    bf16x8_t R, W, K, V, A, B, DO;
    float4_t h0img[2], dhimg[2];   // state at the start of the chunk, adjoint at its end: value tile w, key tiles 2hf, 2hf+1
};

// PART selects which of the eleven 16-byte loads are issued (bit i of the mask): the prefetch is spread
// over the tail of the previous chunk, a few loads at a time, because a wave that issues all of them at
// once sits at the issue stage until the memory pipeline has taken them.
template <unsigned PART, bool PACKED>
__device__ __forceinline__
void load_chunk_inputs(ChunkInputs& in, int n, int lane, const bf16_t* __restrict__ r_, const bf16_t* __restrict__ w_,
                       const bf16_t* __restrict__ k_, const bf16_t* __restrict__ v_,
                       const bf16_t* __restrict__ a_, const bf16_t* __restrict__ b_,
                       const bf16_t* __restrict__ dO_, const float* __restrict__ hs,
                       const float* __restrict__ dhs, const SeqLayout& L)
{
    const int wid = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int w = wid & 3, hf = wid >> 2;
    const int x = lane & 15, g = lane >> 4;
    const ChunkCoord cc = chunk_coord<PACKED>(L, n);   // recomputed wherever it is needed: scalar work, no registers held
    const int H = L.H;
    const int t = cc.c * CH + 16 * w + x;
    // rows past the sequence's end (last chunk only) are read from the last valid row; the consumer zeroes them
    const int64_t row_ld = ((cc.tok0 + (t < cc.len ? t : cc.len - 1)) * H + cc.hi) * HEAD + 32 * hf + 8 * g;
    const int64_t img = cc.rec * 4096 + ((w * 4 + 2 * hf) * 64 + lane) * 4;
    if constexpr (PART & 1u) in.h0img[0] = *reinterpret_cast<const float4_t*>(hs + img);
    if constexpr (PART & 2u) in.h0img[1] = *reinterpret_cast<const float4_t*>(hs + img + 256);
    if constexpr (PART & 4u) in.dhimg[0] = *reinterpret_cast<const float4_t*>(dhs + img);
    if constexpr (PART & 8u) in.dhimg[1] = *reinterpret_cast<const float4_t*>(dhs + img + 256);
    if constexpr (PART & 16u) in.W = *reinterpret_cast<const bf16x8_t*>(w_ + row_ld);
    if constexpr (PART & 32u) in.R = *reinterpret_cast<const bf16x8_t*>(r_ + row_ld);
    if constexpr (PART & 64u) in.K = *reinterpret_cast<const bf16x8_t*>(k_ + row_ld);
    if constexpr (PART & 128u) in.V = *reinterpret_cast<const bf16x8_t*>(v_ + row_ld);
    if constexpr (PART & 256u) in.A = *reinterpret_cast<const bf16x8_t*>(a_ + row_ld);
    if constexpr (PART & 512u) in.B = *reinterpret_cast<const bf16x8_t*>(b_ + row_ld);
    if constexpr (PART & 1024u) {
        if (dO_ != nullptr) in.DO = *reinterpret_cast<const bf16x8_t*>(dO_ + row_ld);
        else in.DO = zero_frag();
    }
    // nothing here looks at the loaded values
}

// Two instantiations.  GENERAL = false (chunk_bwd_kernel) is launched over all chunks and handles those whose decay fits
// one exponent bucket (RWKV7's own range); a chunk that needs several buckets only appends its id to
// `list` ([0] = count, then ids) and leaves.  GENERAL = true (chunk_bwd_general_kernel) is launched afterwards with a small grid,
// walks that list and does the bucket-by-bucket passes.  Kept apart, the rare path's register needs
// do not cost the common one its registers (together they spilled 60 of them).
template <bool GENERAL, bool PACKED>
__device__ __forceinline__
void chunk_bwd_body(int n, int lane, const ChunkInputs& in, ChunkInputs& next, int n_next,
                    const bf16_t* __restrict__ r_, const bf16_t* __restrict__ w_,
                      const bf16_t* __restrict__ k_, const bf16_t* __restrict__ v_,
                      const bf16_t* __restrict__ a_, const bf16_t* __restrict__ b_,
                      const bf16_t* __restrict__ dO_, const float* __restrict__ hs,
                      const float* __restrict__ dhs,
                      bf16_t* __restrict__ dr_, bf16_t* __restrict__ dw_, bf16_t* __restrict__ dk_,
                      bf16_t* __restrict__ dv_, bf16_t* __restrict__ da_, bf16_t* __restrict__ db_,
                      const SeqLayout& L, unsigned* __restrict__ list)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int wid = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int w = wid & 3, hf = wid >> 2;
    const int x = lane & 15, g = lane >> 4;
    const ChunkCoord cc = chunk_coord<PACKED>(L, n);
    const int H = L.H, c = cc.c, hi = cc.hi;
    const int T = cc.len;              // of this chunk's sequence
    const int t_local = 16 * w + x;
    const int t = c * CH + t_local;
    const bool valid = t < T;
    const int64_t row = ((cc.tok0 + t) * H + hi) * HEAD;
    const int ch0 = 32 * hf + 8 * g;          // first of this lane's eight channels in the load layout
    const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};

    // Waits until the next chunk's inputs have landed: a use that the compiler must honour.  Not under the condition of
    // the requests themselves: the compiler does not see that the two conditions agree, and a path with requests but
    // without this wait would keep them "in flight" up to the loop's back edge.
    auto collect_next = [&]() {
        asm volatile("" :: "v"(next.R), "v"(next.W), "v"(next.K), "v"(next.V), "v"(next.A), "v"(next.B), "v"(next.DO),
                     "v"(next.h0img[0]), "v"(next.h0img[1]), "v"(next.dhimg[0]), "v"(next.dhimg[1]));
    };
    auto prefetch_next = [&](auto part) {
        if (n_next >= 0)
            load_chunk_inputs<decltype(part)::value, PACKED>(next, n_next, lane, r_, w_, k_, v_, a_, b_, dO_, hs, dhs, L);
    };
    // Six small groups, each issued in a phase of its own: two groups in one phase cost 3 % of the call (a wave sits at
    // the issue stage until the memory pipeline has taken its requests), and none in the phases of the inverse and of
    // M^T, whose waves are the critical path.
    using P1 = std::integral_constant<unsigned, 0x00fu>;      // the two float images
    using P2 = std::integral_constant<unsigned, 0x030u>;      // w, r
    using P3 = std::integral_constant<unsigned, 0x040u>;      // k
    using P4 = std::integral_constant<unsigned, 0x180u>;      // v, a
    using P5 = std::integral_constant<unsigned, 0x200u>;      // b
    using P6 = std::integral_constant<unsigned, 0x400u>;      // dO
    using PALL = std::integral_constant<unsigned, 0x7ffu>;
    const float4_t h0img[2] = {in.h0img[0], in.h0img[1]}, dhimg[2] = {in.dhimg[0], in.dhimg[1]};

    // ---- prologue (as in chunk_summary_kernel): cumulative log decay, scaled operands
    bf16x8_t R = in.R, K = in.K, V = in.V, A = in.A, B = in.B, DO = in.DO;
    if ((c + 1) * CH > T) {            // uniform: only the last chunk of a sequence can be ragged
        if (!valid) {
            const bf16x8_t z = zero_frag();
            R = K = V = A = B = DO = z;
        }
    }
    float gl[8], gstep[8], gsum[8];
    const float vmask = valid ? 1.f : 0.f;     // (times zero rather than a select: no branch around each evaluation)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float wv = (float)in.W[e];
        gstep[e] = vmask * fmaxf(-LOG2E * ex2(LOG2E * wv), G_MIN2);           // log2 of exp(-exp(w))
        gl[e] = row_inclusive_scan(gstep[e]);
    }
    float* tot = reinterpret_cast<float*>(smem + OFF_TOT);
    if (x == 15) {
        float4_t* dst = reinterpret_cast<float4_t*>(tot + w * 64 + ch0);
        dst[0] = float4_t{gl[0], gl[1], gl[2], gl[3]};
        dst[1] = float4_t{gl[4], gl[5], gl[6], gl[7]};
    }
    __syncthreads();
    float xmax = 0.f;
    {
        float pre[8], gother[8];               // gother: chunk totals of the other half's channels (for npass)
#pragma unroll
        for (int e = 0; e < 8; ++e) { pre[e] = 0.f; gsum[e] = 0.f; gother[e] = 0.f; }
#pragma unroll
        for (int ww = 0; ww < 4; ++ww) {
            const float4_t* src = reinterpret_cast<const float4_t*>(tot + ww * 64 + ch0);
            const float4_t* oth = reinterpret_cast<const float4_t*>(tot + ww * 64 + (ch0 ^ 32));
            const float4_t a0 = src[0], a1 = src[1], o0 = oth[0], o1 = oth[1];
            const float vals[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
            const float ovals[8] = {o0.x, o0.y, o0.z, o0.w, o1.x, o1.y, o1.z, o1.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                gsum[j] += vals[j];
                gother[j] += ovals[j];
                if (ww < w) pre[j] += vals[j];
            }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) { gl[e] += pre[e]; xmax = fmaxf(xmax, fmaxf(-gsum[e], -gother[e])); }
    }
    xmax = max_over_rows(xmax);
    const int npass = (int)(xmax * (1.f / BUCKET2)) + 1;       // uniform over the workgroup
    if constexpr (!GENERAL) {
        if (npass > 1) {
            if (threadIdx.x == 0) list[1 + atomicAdd(list, 1u)] = (unsigned)n;
            prefetch_next(PALL{});
            collect_next();                // (so that no path reaches the loop's back edge with requests in flight)
            return;
        }
    }

    // the raw inputs stay packed (bf16) and are widened where they are used
    auto raw = [](const bf16x8_t& f, int e) { return (float)f[e]; };

    // tile writer for this lane's piece of its token row
    auto put_row = [&](int off, const bf16x8_t& f) {
        *reinterpret_cast<bf16x8_t*>(smem + off + (t_local * LDT + ch0) * 2) = f;
    };
    // operands of decay bucket p:  Qp = r e^{-(x - 64p)} [x >= 64p],  Ap = a e^{-(xe - 64p)} [xe >= 64p],
    // Kp = k e^{x - 64p} [x in bucket p],  Bp likewise;  x = -gi, xe = -ge.
    // The raw operands are arguments: the epilogue loads them again rather than keeping four fragments
    // (and the four scaled ones) in registers through the whole tile algebra.
    auto bucket_operands = [&](int p, const bf16x8_t& R_, const bf16x8_t& K_, const bf16x8_t& A_, const bf16x8_t& B_,
                               bf16x8_t& Qp, bf16x8_t& Ap, bf16x8_t& Kp, bf16x8_t& Bp) {
        if constexpr (!GENERAL) {          // one bucket: every exponent is in range, no selection
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float up = ex2(-gl[e]);
                Kp[e] = (bf16_t)(raw(K_, e) * up);
                Bp[e] = (bf16_t)(raw(B_, e) * up);
                Qp[e] = (bf16_t)(raw(R_, e) * ex2(gl[e]));
                Ap[e] = (bf16_t)(raw(A_, e) * ex2(gl[e] - gstep[e]));
            }
            return;
        }
        const float base = BUCKET2 * (float)p;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float xi = -gl[e], xe = xi + gstep[e];
            const float up = (xi >= base && xi < base + BUCKET2) ? ex2(xi - base) : 0.f;
            Kp[e] = (bf16_t)(raw(K_, e) * up);
            Bp[e] = (bf16_t)(raw(B_, e) * up);
            Qp[e] = (bf16_t)(xi >= base ? raw(R_, e) * ex2(base - xi) : 0.f);
            Ap[e] = (bf16_t)(xe >= base ? raw(A_, e) * ex2(base - xe) : 0.f);
        }
    };
    auto put_operands = [&](const bf16x8_t& Qp, const bf16x8_t& Ap, const bf16x8_t& Kp, const bf16x8_t& Bp) {
        put_row(S_QG, Qp); put_row(S_AG, Ap); put_row(S_KT, Kp); put_row(S_BT, Bp);
    };
    auto get_row = [&](int off) {
        return *reinterpret_cast<const bf16x8_t*>(smem + off + (t_local * LDT + ch0) * 2);
    };
    // Several buckets: kg, bg rows (bucket-free: exponent G - gi <= 0), kept for the tiles written later and for dG.
    // One bucket: kg = k~ diag(e^G) and bg = b~ diag(e^G) with k~, b~ already in their tiles, so the chunk decay is
    // folded into dh' instead (DECAY_IN_DH): every product with kg or bg takes k~ or b~ against e^G dh', the
    // gradients of kg and bg come out times e^G, which is what dk, db and dG need of them, and no kg / bg tile,
    // no e^{G - gi} and no barrier around their slot is left.
    constexpr bool DECAY_IN_DH = !GENERAL;
    // (slots of the tiles whose place depends on the plan)
    constexpr int T_H0 = DECAY_IN_DH ? S1_H0 : S_H0, T_DH = DECAY_IN_DH ? S1_DH : S_DH;
    constexpr int T_DSA = DECAY_IN_DH ? S1_DSA : S_DSA, T_DAAK = DECAY_IN_DH ? S1_DAAK : S_DAAK;
    bf16x8_t KG, BG;
    {
        bf16x8_t Qp, Ap, Kp, Bp;
        bucket_operands(0, R, K, A, B, Qp, Ap, Kp, Bp);
        put_operands(Qp, Ap, Kp, Bp);
        put_row(S_V, V); put_row(S_DO, DO);
        if constexpr (DECAY_IN_DH) {
            // h0^T tile [v][c] from the float image; wave = (value tile w, key tiles 2hf, 2hf + 1)
#pragma unroll
            for (int m = 0; m < 2; ++m) tile_store_acc(smem, T_H0, w, 2 * hf + m, lane, h0img[m]);
            if (w == 0 && x == 0) {
                float4_t* e4 = reinterpret_cast<float4_t*>(reinterpret_cast<float*>(smem + OFF_EGB) + ch0);
                e4[0] = float4_t{ex2(gsum[0]), ex2(gsum[1]), ex2(gsum[2]), ex2(gsum[3])};
                e4[1] = float4_t{ex2(gsum[4]), ex2(gsum[5]), ex2(gsum[6]), ex2(gsum[7])};
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float tail = ex2(gsum[e] - gl[e]);
                KG[e] = (bf16_t)(raw(K, e) * tail);
                BG[e] = (bf16_t)(raw(B, e) * tail);
            }
        }
    }
    __syncthreads();

    // ---- dh'^T tile [v][c]; the decay part of dG needs  sum_v h0 dh'  in float32
    auto adjoint_tile = [&]() {
        float dgdec[8];                    // partial over this lane's value column, key rows 16(2hf+m)+4g+e
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            float4_t dh = dhimg[m];
            if constexpr (DECAY_IN_DH)
                dh = dh * *reinterpret_cast<const float4_t*>(reinterpret_cast<const float*>(smem + OFF_EGB) + 16 * (2 * hf + m) + 4 * g);
            tile_store_acc(smem, T_DH, w, 2 * hf + m, lane, dh);
#pragma unroll
            for (int e = 0; e < 4; ++e) dgdec[4 * m + e] = h0img[m][e] * dh[e];      // (DECAY_IN_DH: e^G included)
        }
        // reduce over the 16 value columns of the row, then (later) over the 4 value tiles through LDS
        float* red = reinterpret_cast<float*>(smem + OFF_RED);
#pragma unroll
        for (int i = 0; i < 8; ++i) dgdec[i] = row_inclusive_suffix_scan(dgdec[i]);   // lane x = 0: the row's sum
        if (x == 0) {
#pragma unroll
            for (int m = 0; m < 2; ++m)
                *reinterpret_cast<float4_t*>(red + w * 64 + 16 * (2 * hf + m) + 4 * g) =
                    float4_t{dgdec[4 * m], dgdec[4 * m + 1], dgdec[4 * m + 2], dgdec[4 * m + 3]};
        }
    };
    if constexpr (DECAY_IN_DH) adjoint_tile();     // its slot is free from the start, e^G is there since the barrier
    // The next chunk's inputs are requested from here on, a few at a time: this chunk's copies are dead since the
    // prologue, so the requests cost no registers, and they have landed long before they are collected.
    prefetch_next(P1{});

    // ---- G1: block row w (rows j, column i = 16w + x) of Aqk, Aqb (waves hf = 0) and of Aak, Aab
    // (waves hf = 1), bucket by bucket
    float4_t acc1[4], acc2[4];
    float4_t diagX = zero4;
#pragma unroll
    for (int J = 0; J < 4; ++J) { acc1[J] = zero4; acc2[J] = zero4; }
    const int s_qa = hf ? S_AG : S_QG;
    const int np = GENERAL ? npass : 1;
    for (int p = 0; p < np; ++p) {
        if (p > 0) {
            __syncthreads();
            bf16x8_t Qp, Ap, Kp, Bp;
            bucket_operands(p, R, K, A, B, Qp, Ap, Kp, Bp);
            put_operands(Qp, Ap, Kp, Bp);
            __syncthreads();
        }
        const bf16x8_t qa[2] = {tile_rows(smem, s_qa, w, 0, lane), tile_rows(smem, s_qa, w, 1, lane)};
#pragma unroll
        for (int J = 0; J < 4; ++J) {
            if (J <= w) {
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    acc1[J] = mfma_bf16(tile_rows(smem, S_KT, J, s, lane), qa[s], acc1[J]);
                    acc2[J] = mfma_bf16(tile_rows(smem, S_BT, J, s, lane), qa[s], acc2[J]);
                }
            }
        }
        if (hf) {
#pragma unroll
            for (int s = 0; s < 2; ++s)
                diagX = mfma_bf16(qa[s], tile_rows(smem, S_BT, w, s, lane), diagX);
        }
    }
    if (np > 1) {                     // leave the bucket-0 operands in the tiles for the later phases
        __syncthreads();
        bf16x8_t Qp, Ap, Kp, Bp;
        bucket_operands(0, R, K, A, B, Qp, Ap, Kp, Bp);
        put_operands(Qp, Ap, Kp, Bp);
    }
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
        // tiles [i][j]: row i = 16w + x, columns 16J + 4g .. +3 (zero right of the diagonal block)
        tile_store_acc(smem, hf ? S_AAK : S_AQK, w, J, lane, J <= w ? acc1[J] : zero4);
        tile_store_acc(smem, hf ? S_AAB : S_AQB, w, J, lane, J <= w ? acc2[J] : zero4);
    }
    // ---- inverse of the diagonal block (see chunk_summary_kernel); the waves that hold Aab do it
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
    // ---- M^T tile [j][i]: column block J = w, rows i >= j; zero above the diagonal blocks
    if (hf) {
        // Dm: column j' = x, rows i' = 4g+e of Dinv  ->  MT[16w + x][16w + 4g + e]
        tile_store_acc(smem, S_MT, w, w, lane, Dm);
#pragma unroll
        for (int I = 0; I < 4; ++I) if (I < w) tile_store_acc(smem, S_MT, w, I, lane, zero4);
        bf16x4_t Mcol[4];
        Mcol[0] = Mcol[1] = Mcol[2] = Mcol[3] = pack4(zero4);
#pragma unroll
        for (int L = 0; L < 4; ++L) if (L == w) Mcol[L] = pack4(Dm);
#pragma unroll
        for (int I = 1; I < 4; ++I) {
            if (I > w) {
                float4_t S = zero4;
#pragma unroll
                for (int L = 0; L < 3; ++L) {
                    if (L >= w && L < I) {
                        const bf16x4_t a4 = *reinterpret_cast<const bf16x4_t*>(
                            smem + S_AAB + ((16 * I + x) * LDT + 16 * L + 4 * g) * 2);
                        S = mfma_bf16_k16(a4, Mcol[L], S);
                    }
                }
                const bf16x4_t d4 = *reinterpret_cast<const bf16x4_t*>(smem + OFF_DI + I * 512 + (x * 16 + 4 * g) * 2);
                const float4_t Mi = mfma_bf16_k16(d4, pack4(S), zero4);
                Mcol[I] = pack4(Mi);
                tile_store_acc(smem, S_MT, w, I, lane, Mi);     // column j = 16w + x, rows i = 16I + 4g + e
            }
        }
    }
    if constexpr (!DECAY_IN_DH) {
        __syncthreads();                   // Aab is dead from here: its slot takes h0
        // ---- h0^T tile [v][c] from the float image; wave = (value tile w, key tiles 2hf, 2hf + 1)
#pragma unroll
        for (int m = 0; m < 2; ++m) tile_store_acc(smem, T_H0, w, 2 * hf + m, lane, h0img[m]);
        __syncthreads();
    }
    // (one bucket: h0 has been in its tile since the prologue, so Y needs nothing of the M^T phase and the waves
    // that do not take part in it start here; the barrier behind Y publishes M^T as well)

    // generic product: acc[m] += sum_s A(2hf + m, s) * B(s): this wave's two row tiles of its 16 columns
    auto gemm = [&](float4_t (&acc)[2], auto&& Af, auto&& Bf) {
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const bf16x8_t bfrag = Bf(s);
#pragma unroll
            for (int m = 0; m < 2; ++m) acc[m] = mfma_bf16(Af(2 * hf + m, s), bfrag, acc[m]);
        }
    };
    // the same with fragments that are already in registers: operands shared by consecutive products are
    // read from LDS once
    struct FragA { bf16x8_t f[2][2]; };
    struct FragB { bf16x8_t f[2]; };
    auto gemm_rr = [&](float4_t (&acc)[2], const FragA& a, const FragB& b) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int m = 0; m < 2; ++m) acc[m] = mfma_bf16(a.f[m][s], b.f[s], acc[m]);
    };
    auto gemm_ar = [&](float4_t (&acc)[2], auto&& Af, const FragB& b) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int m = 0; m < 2; ++m) acc[m] = mfma_bf16(Af(2 * hf + m, s), b.f[s], acc[m]);
    };
    auto loadA = [&](auto&& Af) {
        FragA a;
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int s = 0; s < 2; ++s) a.f[m][s] = Af(2 * hf + m, s);
        return a;
    };
    auto loadB = [&](auto&& Bf) { FragB b; b.f[0] = Bf(0); b.f[1] = Bf(1); return b; };
    auto rowsA = [&](int off) { return [=](int mt, int s) { return tile_rows(smem, off, mt, s, lane); }; };
    auto colsA = [&](int off) { return [=](int mt, int s) { return tile_cols(smem, off, mt, s, lane); }; };
    auto rowsB = [&](int off) { return [=](int s) { return tile_rows(smem, off, w, s, lane); }; };
    auto colsB = [&](int off) { return [=](int s) { return tile_cols(smem, off, w, s, lane); }; };
    auto clear = [&](float4_t (&acc)[2]) { acc[0] = acc[1] = zero4; };
    auto store_tile = [&](int off, const float4_t (&acc)[2]) {
#pragma unroll
        for (int m = 0; m < 2; ++m) tile_store_acc(smem, off, w, 2 * hf + m, lane, acc[m]);
    };

    float4_t tmp[2];
    // Y[j][v] = ag h0 + Aak V        -> Y^T[v][j]
    clear(tmp);
    gemm(tmp, rowsA(S_AG), rowsB(T_H0));
    gemm(tmp, rowsA(S_AAK), colsB(S_V));
    store_tile(S_Y, tmp);
    __syncthreads();
    // SA[i][v] = M Y                 -> SA^T[v][i]
    clear(tmp);
    gemm(tmp, colsA(S_MT), rowsB(S_Y));
    store_tile(S_SA, tmp);
    __syncthreads();                       // SA is there; Y is dead (general plan: its slot takes dh')

    if constexpr (!DECAY_IN_DH) adjoint_tile();
    if constexpr (!DECAY_IN_DH) {
        put_row(S_BG, BG);
        __syncthreads();
    }

    prefetch_next(P2{});
    // accumulators that live to the end: rows = tokens, column = channel 16w + x
    float4_t acc_q[2], acc_a[2], acc_kg[2], acc_bg[2], acc_v[2];
    clear(acc_q); clear(acc_a); clear(acc_kg); clear(acc_bg); clear(acc_v);
    // dkg[j][c] = V dh'^T ;  dbg[j][c] = SA dh'^T ;  dqg_h[i][c] = dO h0^T
    {
        const FragB DHc = loadB(colsB(T_DH));
        gemm_ar(acc_kg, rowsA(S_V), DHc);
        gemm_ar(acc_bg, colsA(S_SA), DHc);
    }
    gemm(acc_q, rowsA(S_DO), colsB(T_H0));
    prefetch_next(P3{});
    // dSA[j][v] = Aqb^T dO + bg dh'   -> dSA^T[v][j]
    const FragB DOc = loadB(colsB(S_DO)), DHr = loadB(rowsB(T_DH));
    clear(tmp);
    gemm_ar(tmp, colsA(S_AQB), DOc);
    gemm_ar(tmp, rowsA(DECAY_IN_DH ? S_BT : S_BG), DHr);
    store_tile(T_DSA, tmp);
    if constexpr (!DECAY_IN_DH) {
        __syncthreads();                   // bg is dead: its slot takes kg
        put_row(S_KG, KG);
        __syncthreads();
    }
    // dV[j][v] = Aqk^T dO + kg dh' (+ Aak^T dY below)
    gemm_ar(acc_v, colsA(S_AQK), DOc);
    gemm_ar(acc_v, rowsA(DECAY_IN_DH ? S_KT : S_KG), DHr);
    __syncthreads();                       // dSA is there (general plan: dh' is dead, its slot takes dY)
    // dY[j][v] = M^T dSA              -> dY^T[v][j]
    clear(tmp);
    gemm(tmp, rowsA(S_MT), rowsB(T_DSA));
    store_tile(S_DY, tmp);
    __syncthreads();                       // M^T, dSA and kg are dead
    prefetch_next(P4{});
    gemm(acc_v, colsA(S_AAK), rowsB(S_DY));
    gemm(acc_a, colsA(S_DY), colsB(T_H0));         // dag_h[i][c] = dY h0^T
    if constexpr (!DECAY_IN_DH) __syncthreads();   // h0 is dead: its slot takes dAqk (one bucket: dSA's, dead since dY)

    prefetch_next(P5{});
    // ---- dA matrices as tiles [i][j] (column tile w = token tile i; rows of the product are j).  Their
    // slots (h0, M^T, kg, dSA) are dead since the last barrier, so each is stored as soon as it is masked.
    {
        auto masked_store = [&](int off, float4_t (&d)[2], bool strict) {
#pragma unroll
            for (int m = 0; m < 2; ++m) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int jj = 16 * (2 * hf + m) + 4 * g + e, ii = 16 * w + x;
                    if (strict ? jj >= ii : jj > ii) d[m][e] = 0.f;
                }
            }
            store_tile(off, d);
        };
        float4_t d[2];
        const FragA Vr = loadA(rowsA(S_V));
        const FragB DOr = loadB(rowsB(S_DO));
        clear(d); gemm_rr(d, Vr, DOr);  masked_store(S_DAQK, d, false);   // dAqk[i][j] = sum_v V[j][v] dO[i][v]
        const FragA SAc = loadA(colsA(S_SA));
        clear(d); gemm_rr(d, SAc, DOr); masked_store(S_DAQB, d, false);   // dAqb[i][j] = sum_v SA[j][v] dO[i][v]
        const FragB DYc = loadB(colsB(S_DY));
        clear(d); gemm_rr(d, Vr, DYc);  masked_store(T_DAAK, d, true);    // dAak[i][j] = sum_v V[j][v] dY[i][v]
        clear(d); gemm_rr(d, SAc, DYc); masked_store(S_DAAB, d, true);    // dAab[i][j] = sum_v SA[j][v] dY[i][v]
    }
    __syncthreads();

    prefetch_next(P6{});
    // ---- the decay-weighted products and the epilogue in the load layout.
    // dgi / dge are formed from the SAME bf16-rounded operands the products used (z qg - z kt - ...), not
    // from dr r - dk k - db b: the pair terms then cancel exactly in the suffix sum instead of leaving
    // rounding noise of the size of the cancelled terms (this is worth a factor 10 on dw).
    float* st0 = reinterpret_cast<float*>(smem + S_STAGE0);
    float* st1 = reinterpret_cast<float*>(smem + S_STAGE1);
    float* st2 = reinterpret_cast<float*>(smem + S_STAGE2);
    // Staging tiles [channel][token] with the tokens of channel ch rotated by 16 (ch / 8): the four lane groups
    // of a reading wave (channels 8 apart, same tokens) would otherwise all land on the same sixteen banks.
    auto stage_put = [&](float* st, const float4_t (&acc)[2]) {     // [channel 16w+x][token 16mt+4g..]
        const int rot = 16 * (2 * w + (x >> 3));
#pragma unroll
        for (int m = 0; m < 2; ++m)
            *reinterpret_cast<float4_t*>(st + (16 * w + x) * LDZ + ((16 * (2 * hf + m) + 4 * g + rot) & 63)) = acc[m];
    };
    auto stage_get = [&](const float* st, float (&z)[8]) {           // this lane's token, its 8 channels
        const int tr = (t_local + 16 * g) & 63;                      // (ch0 + e) / 8 = 4 hf + g for every e
#pragma unroll
        for (int e = 0; e < 8; ++e) z[e] = st[(ch0 + e) * LDZ + tr];
    };
    auto pack_rows = [&](const float (&val)[8]) {
        bf16x8_t o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (bf16_t)val[e];
        return o;
    };
    auto store_rows = [&](bf16_t* dst, const bf16x8_t& o) {
        if (valid) *reinterpret_cast<bf16x8_t*>(dst + row + ch0) = o;
    };
    // sall = dgi + dge (the suffix-scan input), dge, and dkk = dkg kg + dbg bg (for dG)
    float sall[8], dge[8], dkk[8];
    // (one bucket: the six output stores are spread over the epilogue and the reductions behind it: stores issued
    // back to back hold the wave at the issue stage until the memory pipeline has taken them)
    bf16x8_t late_db, late_dr, late_da;
    if constexpr (!GENERAL) {
        // Common case, one decay bucket: every output is final after one staging round and is stored
        // at once, so only sall / dge / dkk stay live.
        float4_t acc_k[2], acc_b[2];
        clear(acc_k); clear(acc_b);
        {
            // Eight products, software-pipelined by hand: the fragments of the next product are requested before the
            // MFMAs of the current one are issued (the fences keep the compiler from sinking each read next to its
            // use, where every MFMA would wait out an LDS round trip).
            const FragB KTc = loadB(colsB(S_KT));
            FragA f0 = loadA(rowsA(S_DAQK));
            FragA f1 = loadA(rowsA(T_DAAK));
            __builtin_amdgcn_sched_barrier(0);
            gemm_rr(acc_q, f0, KTc);
            const FragB BTc = loadB(colsB(S_BT));
            f0 = loadA(rowsA(S_DAQB));
            __builtin_amdgcn_sched_barrier(0);
            gemm_rr(acc_a, f1, KTc);
            f1 = loadA(rowsA(S_DAAB));
            __builtin_amdgcn_sched_barrier(0);
            gemm_rr(acc_q, f0, BTc);
            const FragB QGc = loadB(colsB(S_QG));
            f0 = loadA(colsA(S_DAQK));
            __builtin_amdgcn_sched_barrier(0);
            gemm_rr(acc_a, f1, BTc);
            f1 = loadA(colsA(S_DAQB));
            __builtin_amdgcn_sched_barrier(0);
            gemm_rr(acc_k, f0, QGc);
            const FragB AGc = loadB(colsB(S_AG));
            f0 = loadA(colsA(T_DAAK));
            __builtin_amdgcn_sched_barrier(0);
            gemm_rr(acc_b, f1, QGc);
            f1 = loadA(colsA(S_DAAB));
            __builtin_amdgcn_sched_barrier(0);
            gemm_rr(acc_k, f0, AGc);
            __builtin_amdgcn_sched_barrier(0);
            gemm_rr(acc_b, f1, AGc);
        }
        // this lane's pieces of the bucket-0 operands, back from their tiles
        const bf16x8_t Qp = get_row(S_QG), Ap = get_row(S_AG), Kp = get_row(S_KT), Bp = get_row(S_BT);
        // Every tile is dead now, so all seven accumulator sets change layout in one round: float
        // tiles [channel][token] over the whole tile area, one barrier before and one after.
        __syncthreads();
        auto stg = [&](int i) { return reinterpret_cast<float*>(smem + i * (64 * LDZ * 4)); };
        stage_put(stg(0), acc_k); stage_put(stg(1), acc_kg); stage_put(stg(2), acc_v);
        stage_put(stg(3), acc_b); stage_put(stg(4), acc_bg); stage_put(stg(5), acc_q); stage_put(stg(6), acc_a);
        __syncthreads();
        float zk[8], zkg[8], zv[8], zb[8], zbg[8], zq[8], za[8];
        stage_get(stg(0), zk); stage_get(stg(1), zkg); stage_get(stg(2), zv);
        stage_get(stg(3), zb); stage_get(stg(4), zbg); stage_get(stg(5), zq); stage_get(stg(6), za);
        float out[8];
        // Every request for the next chunk's inputs is collected HERE, before the first store below.  On gfx9 loads and
        // stores share one in-flight counter and may complete out of order, so with both kinds outstanding the only wait
        // the compiler can emit for a loaded register is "everything, stores included": left to the loop's back edge, that
        // wait exposed the full latency of the six output stores once per chunk (12 % of the call).
        collect_next();
        float ek[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) ek[e] = ex2(-gl[e]);
        // dk = dkt e^{-gi} + dkg e^{G-gi}, dv.  zkg, zbg are the gradients of kg, bg times e^G (the decay went
        // into dh'): e^G dkg e^{-gi} is the second term, and dkg kg = (e^G dkg) k~.
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            out[e] = (zk[e] + zkg[e]) * ek[e];
            sall[e] = -zk[e] * (float)Kp[e];
            dkk[e] = zkg[e] * (float)Kp[e];
        }
        store_rows(dk_, pack_rows(out));
        // db, dr
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            out[e] = (zb[e] + zbg[e]) * ek[e];
            sall[e] -= zb[e] * (float)Bp[e];
            dkk[e] += zbg[e] * (float)Bp[e];
        }
        late_db = pack_rows(out);
        store_rows(dv_, pack_rows(zv));
#pragma unroll
        for (int e = 0; e < 8; ++e) { out[e] = zq[e] * ex2(gl[e]); sall[e] += zq[e] * (float)Qp[e]; }
        late_dr = pack_rows(out);
        // da
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            out[e] = za[e] * ex2(gl[e] - gstep[e]);
            dge[e] = za[e] * (float)Ap[e];
            sall[e] += dge[e] - dkk[e];
        }
        late_da = pack_rows(out);
        store_rows(db_, late_db);
    } else {
        // Several decay buckets (strong decays): one pass of the products per bucket, each with its own
        // exponent offset, accumulated in registers.
        float dr[8], da[8], dk[8], db[8], dgi[8];
        bf16x8_t R2, K2, A2, B2, Qp, Ap, Kp, Bp;
        {
            const int64_t row_ld = (valid ? row : ((cc.tok0 + (T - 1)) * H + hi) * HEAD) + ch0;
            R2 = *reinterpret_cast<const bf16x8_t*>(r_ + row_ld);
            K2 = *reinterpret_cast<const bf16x8_t*>(k_ + row_ld);
            A2 = *reinterpret_cast<const bf16x8_t*>(a_ + row_ld);
            B2 = *reinterpret_cast<const bf16x8_t*>(b_ + row_ld);
            if (!valid) R2 = K2 = A2 = B2 = zero_frag();
        }
        Qp = get_row(S_QG); Ap = get_row(S_AG); Kp = get_row(S_KT); Bp = get_row(S_BT);
#pragma unroll
        for (int e = 0; e < 8; ++e) { dr[e] = 0.f; da[e] = 0.f; dk[e] = 0.f; db[e] = 0.f; dgi[e] = 0.f; dge[e] = 0.f; dkk[e] = 0.f; }
        {   // dkg, dbg and dV are complete: move them to the load layout now and free their accumulators
            float z[8];
            stage_put(st0, acc_kg); stage_put(st1, acc_bg); stage_put(st2, acc_v);
            __syncthreads();
            stage_get(st0, z);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                dk[e] += z[e] * ex2(gsum[e] - gl[e]);
                dkk[e] += z[e] * (float)KG[e];
            }
            stage_get(st1, z);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                db[e] += z[e] * ex2(gsum[e] - gl[e]);
                dkk[e] += z[e] * (float)BG[e];
            }
            stage_get(st2, z);
            store_rows(dv_, pack_rows(z));
        }
        for (int p = 0; p < npass; ++p) {
            float4_t acc_k[2], acc_b[2];
            clear(acc_k); clear(acc_b);
            if (p > 0) {
                clear(acc_q); clear(acc_a);
                __syncthreads();
                bucket_operands(p, R2, K2, A2, B2, Qp, Ap, Kp, Bp);
                put_operands(Qp, Ap, Kp, Bp);
                __syncthreads();
            }
            gemm(acc_q, rowsA(S_DAQK), colsB(S_KT)); gemm(acc_q, rowsA(S_DAQB), colsB(S_BT));
            gemm(acc_a, rowsA(S_DAAK), colsB(S_KT)); gemm(acc_a, rowsA(S_DAAB), colsB(S_BT));
            gemm(acc_k, colsA(S_DAQK), colsB(S_QG)); gemm(acc_k, colsA(S_DAAK), colsB(S_AG));
            gemm(acc_b, colsA(S_DAQB), colsB(S_QG)); gemm(acc_b, colsA(S_DAAB), colsB(S_AG));
            const float base = BUCKET2 * (float)p;
            float z[8];
            __syncthreads();               // V, dO, Aqk, Aqb, Aak, dY, SA slots are free for staging
            stage_put(st0, acc_q); stage_put(st1, acc_a); stage_put(st2, acc_k);
            __syncthreads();
            stage_get(st0, z);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float xi = -gl[e];
                dr[e] += xi >= base ? z[e] * ex2(base - xi) : 0.f;
                dgi[e] += z[e] * (float)Qp[e];
            }
            stage_get(st1, z);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float xe = -gl[e] + gstep[e];
                da[e] += xe >= base ? z[e] * ex2(base - xe) : 0.f;
                dge[e] += z[e] * (float)Ap[e];
            }
            stage_get(st2, z);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float xi = -gl[e];
                dk[e] += (xi >= base && xi < base + BUCKET2) ? z[e] * ex2(xi - base) : 0.f;
                dgi[e] -= z[e] * (float)Kp[e];
            }
            __syncthreads();
            stage_put(st0, acc_b);
            __syncthreads();
            stage_get(st0, z);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float xi = -gl[e];
                db[e] += (xi >= base && xi < base + BUCKET2) ? z[e] * ex2(xi - base) : 0.f;
                dgi[e] -= z[e] * (float)Bp[e];
            }
        }
        store_rows(dr_, pack_rows(dr)); store_rows(dk_, pack_rows(dk)); store_rows(da_, pack_rows(da)); store_rows(db_, pack_rows(db));
#pragma unroll
        for (int e = 0; e < 8; ++e) sall[e] = dgi[e] - dkk[e] + dge[e];
    }
    // dG = e^G sum_v(h0 dh') + sum over the 64 tokens of dkk;  dg = suffix_sum(dgi + dge) - dge + dG
    float dg[8];
    {
        float* red = reinterpret_cast<float*>(smem + OFF_RED);     // [4 value tiles][64]: sum_v h0 dh' partials
        float* red2 = red + 256;                                    // [4 token tiles][64]: token partial sums
        float sfx[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            sfx[e] = row_inclusive_suffix_scan(sall[e]);            // over this wave's 16 tokens
            dkk[e] = row_inclusive_suffix_scan(dkk[e]);             // lane x = 0: sum over the wave's 16 tokens
        }
        if constexpr (!GENERAL) store_rows(dr_, late_dr);
        float* totw = reinterpret_cast<float*>(smem + OFF_TOT);     // [4 token tiles][64]: tile totals of dgi+dge
        if (x == 0) {                                               // token 0 of the tile holds the tile totals
            float4_t* t4 = reinterpret_cast<float4_t*>(totw + w * 64 + ch0);
            float4_t* r4 = reinterpret_cast<float4_t*>(red2 + w * 64 + ch0);
            t4[0] = float4_t{sfx[0], sfx[1], sfx[2], sfx[3]}; t4[1] = float4_t{sfx[4], sfx[5], sfx[6], sfx[7]};
            r4[0] = float4_t{dkk[0], dkk[1], dkk[2], dkk[3]}; r4[1] = float4_t{dkk[4], dkk[5], dkk[6], dkk[7]};
        }
        __syncthreads();
        if constexpr (!GENERAL) store_rows(da_, late_da);
        float later[8], dGs[8], dec[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) { later[e] = 0.f; dGs[e] = 0.f; dec[e] = 0.f; }
#pragma unroll
        for (int ww = 0; ww < 4; ++ww) {
            const float4_t* t4 = reinterpret_cast<const float4_t*>(totw + ww * 64 + ch0);
            const float4_t* r4 = reinterpret_cast<const float4_t*>(red2 + ww * 64 + ch0);
            const float4_t* d4 = reinterpret_cast<const float4_t*>(red + ww * 64 + ch0);
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                const float4_t tv = t4[hh], rv = r4[hh], dv = d4[hh];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (ww > w) later[4 * hh + j] += tv[j];
                    dGs[4 * hh + j] += rv[j];
                    dec[4 * hh + j] += dv[j];
                }
            }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e)
            dg[e] = sfx[e] + later[e] - dge[e] + dGs[e] + (DECAY_IN_DH ? dec[e] : ex2(gsum[e]) * dec[e]);
    }
    {
        float dwv[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) dwv[e] = dg[e] * (LN2 * gstep[e]);     // d/dw of g = -exp(w) is g itself
        store_rows(dw_, pack_rows(dwv));
    }
}

#define RWKV7_BWD_PARAMS \
    const bf16_t* __restrict__ r_, const bf16_t* __restrict__ w_, const bf16_t* __restrict__ k_, \
    const bf16_t* __restrict__ v_, const bf16_t* __restrict__ a_, const bf16_t* __restrict__ b_, \
    const bf16_t* __restrict__ dO_, const float* __restrict__ hs, const float* __restrict__ dhs, \
    bf16_t* __restrict__ dr_, bf16_t* __restrict__ dw_, bf16_t* __restrict__ dk_, bf16_t* __restrict__ dv_, \
    bf16_t* __restrict__ da_, bf16_t* __restrict__ db_, SeqLayout L, unsigned* __restrict__ list
#define RWKV7_BWD_ARGS r_, w_, k_, v_, a_, b_, dO_, hs, dhs, dr_, dw_, dk_, dv_, da_, db_, L, list

// One workgroup fits a CU, so the grid is one workgroup per CU, each walking chunks n, n + grid, ...
// with the next chunk's inputs in flight during the current chunk's last third.
// (PACKED: compiled apart for layouts with and without cumulative lengths -- with the choice made at run
// time the dense case ran 12 % slower.)
template <bool PACKED>
__global__ __launch_bounds__(512, 1) void chunk_bwd_kernel(RWKV7_BWD_PARAMS) {
    // chunks in all: with packed sequences the number of listed chunks times H
    const int total = !PACKED ? L.B * L.H * ((L.T + CH - 1) / CH) : load_table(L.items) * L.H;
    int n = blockIdx.x;
    if (n >= total) return;
    ChunkInputs cur;
    load_chunk_inputs<0x7ffu, PACKED>(cur, n, (int)(threadIdx.x & 63), r_, w_, k_, v_, a_, b_, dO_, hs, dhs, L);
    // The first chunk's inputs are waited for in front of the loop: with requests in flight at the loop's entry and
    // stores in flight at its back edge, the compiler has to wait for "everything" at the loop's top, which on the
    // back edge means the previous chunk's output stores (see chunk_bwd_body).
    asm volatile("" :: "v"(cur.R), "v"(cur.W), "v"(cur.K), "v"(cur.V), "v"(cur.A), "v"(cur.B), "v"(cur.DO),
                 "v"(cur.h0img[0]), "v"(cur.h0img[1]), "v"(cur.dhimg[0]), "v"(cur.dhimg[1]));
    while (true) {
        // the lane id is made opaque per iteration so that per-lane addresses are recomputed where they
        // are used instead of being hoisted out of the loop and kept in registers
        int lane = threadIdx.x & 63;
        asm volatile("" : "+v"(lane));
        const int n_next = n + (int)gridDim.x < total ? n + (int)gridDim.x : -1;
        ChunkInputs next;
        chunk_bwd_body<false, PACKED>(n, lane, cur, next, n_next, RWKV7_BWD_ARGS);
        if (n_next < 0) break;
        cur = next;
        n = n_next;
        __syncthreads();                       // the next chunk reuses every tile
    }
}

// a few workgroups walking the list of chunks that need several decay buckets
template <bool PACKED>
__global__ __launch_bounds__(512, 1) void chunk_bwd_general_kernel(RWKV7_BWD_PARAMS) {
    const unsigned count = list[0];
    for (unsigned it = blockIdx.x; it < count; it += gridDim.x) {
        int lane = threadIdx.x & 63;
        asm volatile("" : "+v"(lane));         // as in chunk_bwd_kernel
        const int n = (int)list[1 + it];
        ChunkInputs cur;
        load_chunk_inputs<0x7ffu, PACKED>(cur, n, lane, r_, w_, k_, v_, a_, b_, dO_, hs, dhs, L);
        ChunkInputs unused;
        chunk_bwd_body<true, PACKED>(n, lane, cur, unused, -1, RWKV7_BWD_ARGS);
        __syncthreads();                       // the next chunk reuses every tile
    }
}

}  // namespace

size_t bwd_chunk_workspace_bytes(int B, int T, int H, bool varlen) {
    const int64_t nchunks = chunk_records(B, T, H, varlen);
    // pp, qc, Qt^T dO: 4096 bf16 each; eg: 64 float; hs, dhs: 4096 float each; then the list of
    // chunks that need several decay buckets (a count and up to nchunks ids)
    return (size_t)(nchunks * (3 * 4096 * 2 + 64 * 4 + 2 * 4096 * 4) + (nchunks + 1) * 4) +
           (varlen ? chunk_items_bytes(B, T) : 0);
}

namespace {
template <bool PACKED>
hipError_t launch_chunk_bwd_kernels(const BwdArgs& p, const SeqLayout& L, int64_t nchunks, const float* hs,
                                    const float* dhs, unsigned* list, hipStream_t stream) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(chunk_bwd_kernel<PACKED>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, BWD_LDS_BYTES);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(chunk_bwd_general_kernel<PACKED>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, BWD_LDS_BYTES);
    if (e != hipSuccess) return e;
    int dev = 0, cus = 0;
    e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return e;
    const unsigned pgrid = (unsigned)(nchunks < cus ? nchunks : cus);
    chunk_bwd_kernel<PACKED><<<dim3(pgrid), dim3(512), BWD_LDS_BYTES, stream>>>(
        (const bf16_t*)p.r, (const bf16_t*)p.w, (const bf16_t*)p.k, (const bf16_t*)p.v,
        (const bf16_t*)p.a, (const bf16_t*)p.b, (const bf16_t*)p.dO, hs, dhs,
        (bf16_t*)p.dr, (bf16_t*)p.dw, (bf16_t*)p.dk, (bf16_t*)p.dv, (bf16_t*)p.da, (bf16_t*)p.db,
        L, list);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    // the chunks that asked for the bucket-by-bucket passes (usually none: the workgroups read a zero count and leave)
    const unsigned ggrid = (unsigned)(nchunks < 256 ? nchunks : 256);
    chunk_bwd_general_kernel<PACKED><<<dim3(ggrid), dim3(512), BWD_LDS_BYTES, stream>>>(
        (const bf16_t*)p.r, (const bf16_t*)p.w, (const bf16_t*)p.k, (const bf16_t*)p.v,
        (const bf16_t*)p.a, (const bf16_t*)p.b, (const bf16_t*)p.dO, hs, dhs,
        (bf16_t*)p.dr, (bf16_t*)p.dw, (bf16_t*)p.dk, (bf16_t*)p.dv, (bf16_t*)p.da, (bf16_t*)p.db,
        L, list);
    return hipGetLastError();
}
}  // namespace

hipError_t launch_bwd_chunk(const BwdArgs& p, void* ws, hipStream_t stream) {
    const int64_t nchunks = chunk_records(p.B, p.T, p.H, p.cu != nullptr);
    unsigned char* base = static_cast<unsigned char*>(ws) + (p.cu ? chunk_items_bytes(p.B, p.T) : 0);
    bf16_t* pp = reinterpret_cast<bf16_t*>(base);
    bf16_t* qc = reinterpret_cast<bf16_t*>(base + nchunks * 8192);
    bf16_t* qdo = reinterpret_cast<bf16_t*>(base + nchunks * 16384);
    float* hs = reinterpret_cast<float*>(base + nchunks * 24576);
    float* dhs = reinterpret_cast<float*>(base + nchunks * 40960);
    float* eg = reinterpret_cast<float*>(base + nchunks * 57344);
    unsigned* list = reinterpret_cast<unsigned*>(base + nchunks * (57344 + 256));

    SeqArgs f;
    f.r = p.r; f.w = p.w; f.k = p.k; f.v = p.v; f.a = p.a; f.b = p.b;
    f.h0 = p.h0; f.h0_batch_stride = p.h0_batch_stride; f.h0_map = nullptr; f.n_state = 0; f.ht_in_place = false; f.o = nullptr; f.ht = nullptr;
    f.B = p.B; f.T = p.T; f.H = p.H; f.N = HEAD; f.dtype = p.dtype; f.cu = p.cu; f.u6 = nullptr;
    const SeqLayout L = seq_layout(f, ws);
    hipError_t e = hipSuccess;
    if (p.cu != nullptr) {
        TailFill tail{};
        tail.p[0] = p.dr; tail.p[1] = p.dw; tail.p[2] = p.dk; tail.p[3] = p.dv; tail.p[4] = p.da; tail.p[5] = p.db;
        tail.n = 6; tail.row_bytes = (int64_t)p.H * HEAD * 2;
        e = launch_chunk_items(L, ws, nullptr, 0, nullptr, tail, stream);
    }
    if (e != hipSuccess) return e;
    e = launch_bwd_summary(f, L, p.dO, qdo, pp, qc, eg, stream);
    if (e != hipSuccess) return e;
    const unsigned BH = (unsigned)(p.B * p.H);
    chunk_scans_kernel<<<dim3(2 * BH), dim3(256), 2 * SCAN2_STAGE_BYTES, stream>>>(pp, qc, qdo, eg, p.h0, p.h0_batch_stride, p.dht,
                                                               hs, dhs, p.dh0, L, list);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    return p.cu != nullptr ? launch_chunk_bwd_kernels<true>(p, L, nchunks, hs, dhs, list, stream)
                           : launch_chunk_bwd_kernels<false>(p, L, nchunks, hs, dhs, list, stream);
}

}  // namespace rwkv7
