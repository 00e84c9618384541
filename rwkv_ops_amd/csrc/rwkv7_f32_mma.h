// What the float32 chunk kernels (16-token chunks on the float32 matrix cores, K = V = 64) share: the register
// layouts are described at the top of rwkv7_fwd_chunk_f32.hip.
#pragma once
#include "rwkv7_chunk.h"
#include "rwkv7_common.h"

namespace rwkv7 {

constexpr int C16 = 16;                        // tokens per chunk
constexpr int NH = 64;                         // head size
constexpr float LOG2E = 1.4426950408889634f;
constexpr float G_MIN2 = G_MIN * LOG2E;        // per-step log-decay clamp, in base-2 units
// A chunk whose total log decay exceeds this (in some channel) is walked token by token: k e^{-gi} must stay
// well inside float32 (e^60 times |k|); RWKV7's own decay range gives at most 16 * 0.607 = 9.7.
constexpr float STRONG2 = 60.f * LOG2E;
__device__ __forceinline__ float ex2(float x) { return __builtin_amdgcn_exp2f(x); }

constexpr int LDF = 68;                        // row stride (floats) of the row-major tiles [16 tokens][64 channels]
constexpr int TILE_F = C16 * LDF * 4;          // bytes of a row-major tile

__device__ __forceinline__ float4_t mfma_f32(float a, float b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}
// sum over the 16 lanes of a DPP row, delivered to all of them
__device__ __forceinline__ float row_sum(float x) {
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x121, 0xf, 0xf, true));   // row_ror:1
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x122, 0xf, 0xf, true));   // row_ror:2
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x124, 0xf, 0xf, true));   // row_ror:4
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x128, 0xf, 0xf, true));   // row_ror:8
    return x;
}
// row `row`, columns col .. col + 3 of a tile
__device__ __forceinline__ float4_t tile4(const unsigned char* smem, int off, int row, int col) {
    return *reinterpret_cast<const float4_t*>(smem + off + (row * LDF + col) * 4);
}

// A wave's 64 x 16 part of a state (four accumulator tiles: tile ct = rows 16 ct + 4 g + e of the wave's column x)
// against row-major [key][value] global memory: lane by lane that is sixteen 4-byte accesses, so it goes through a
// [64][LDV] staging area of the wave's own in LDS and leaves / arrives as four 16-byte accesses (row 16 i + lane / 4,
// sixteen bytes lane % 4 of the wave's 64-byte piece of the row).
constexpr int LDV = 20;
constexpr int STAGE_BYTES = NH * LDV * 4;
__device__ __forceinline__ void state_cols_store(float* __restrict__ dst, const float4_t (&t)[4], float* stage, int lane) {
    const int x = lane & 15, g = lane >> 4;
#pragma unroll
    for (int ct = 0; ct < 4; ++ct)
#pragma unroll
        for (int e = 0; e < 4; ++e) stage[(16 * ct + 4 * g + e) * LDV + x] = t[ct][e];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = 16 * i + (lane >> 2), piece = 4 * (lane & 3);
        *reinterpret_cast<float4_t*>(dst + row * NH + piece) = *reinterpret_cast<const float4_t*>(stage + row * LDV + piece);
    }
}
__device__ __forceinline__ void state_cols_request(float4_t (&q)[4], const float* __restrict__ src, int lane) {
#pragma unroll
    for (int i = 0; i < 4; ++i) q[i] = *reinterpret_cast<const float4_t*>(src + (16 * i + (lane >> 2)) * NH + 4 * (lane & 3));
}
__device__ __forceinline__ void state_cols_unpack(float4_t (&t)[4], const float4_t (&q)[4], float* stage, int lane) {
    const int x = lane & 15, g = lane >> 4;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        *reinterpret_cast<float4_t*>(stage + (16 * i + (lane >> 2)) * LDV + 4 * (lane & 3)) = q[i];
#pragma unroll
    for (int ct = 0; ct < 4; ++ct)
#pragma unroll
        for (int e = 0; e < 4; ++e) t[ct][e] = stage[(16 * ct + 4 * g + e) * LDV + x];
}

// Workspace records of the float32 backward, one per 16-token chunk and head.  Dense batches: record
// (b H + h) NT + c.  Packed sequences: sequence b owns the slots from (first row / 16) + b on -- at most
// len / 16 + 1 of them, never overlapping the next sequence's -- and the record of its chunk c is (slot + c) H + h;
// (T_total / 16 + n_seq) H records in all.
struct ChunkRecords {
    int64_t first; int step;           // record of chunk c: first + c * step
    __device__ __forceinline__ int64_t operator()(int c) const { return first + (int64_t)c * step; }
};
__device__ __forceinline__ ChunkRecords f32_chunk_records(const SeqLayout& L, const SeqSpan& sp, int bi, int hi, int nt) {
    if (L.cu == nullptr) return ChunkRecords{((int64_t)bi * L.H + hi) * nt, 1};
    return ChunkRecords{((sp.tok0 >> 4) + bi) * L.H + hi, L.H};
}

}  // namespace rwkv7
