// Shared device helpers for the gfx950 RWKV7 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rwkv7 {

constexpr int HEAD = 64;            // K = V = 64
constexpr int STATE = HEAD * HEAD;  // floats per (batch, head) state

typedef __bf16 bf16_t;
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) {
    return __uint_as_float(bits16 << 16);
}

// decay of one step from the API's `w` argument: exp(-exp(w)).
// v_exp_f32 gives exactly 1.0f at -0.0f, so w = -1e9 (the padding convention)
// yields a decay of exactly 1.
__device__ __forceinline__ float decay_from_w(float w) { return __expf(-__expf(w)); }
// the log decay g = -exp(w)
__device__ __forceinline__ float log_decay_from_w(float w) { return -__expf(w); }

// index of the initial state that batch row `bi` starts from: the row itself, or the (clamped) entry of
// a gather map
__device__ __forceinline__ int64_t state_row(const int* map, int n_state, int bi) {
    if (map == nullptr) return bi;
    const int m = map[bi];
    return m < 0 ? 0 : (m >= n_state ? n_state - 1 : m);
}

// Where the tokens of sequence `bi` lie.  Without `cu`: B sequences of T tokens each, token t of sequence
// bi in row bi * T + t.  With `cu` (cumulative sequence lengths [B + 1], the FlashAttention convention):
// one packed row of T tokens in all, sequence bi = rows cu[bi] .. cu[bi + 1] - 1.  What is read from cu is
// clamped into [0, T] and the end to at least the start, so no value in it can send an access outside the
// tensors (overlapping or unordered entries give meaningless results, not faults).
// Division of an index below 2^31 by a divisor that is fixed per launch, as one 64-bit multiply and a shift
// (the host prepares the multiplier: mul = ceil(2^(31 + sh) / d), sh = ceil(log2 d); exact for every n < 2^31).
// An integer division by a run-time value costs about 25 scalar instructions on gfx950, and the chunk kernels
// take three of them per chunk coordinate.
struct FastDiv { uint32_t mul, sh, d; };
inline FastDiv make_fast_div(uint32_t d) {
    FastDiv f;
    f.d = d; f.sh = 0;
    while ((1ull << f.sh) < d) ++f.sh;
    f.mul = (uint32_t)(((1ull << (31 + f.sh)) + d - 1) / d);
    return f;
}
__device__ __forceinline__ int fast_div(int n, const FastDiv& f) {
    return (int)(((uint64_t)(uint32_t)n * f.mul) >> (31 + f.sh));
}

struct SeqLayout {
    const int* cu;       // nullable, device memory
    const int* items;    // with cu, chunked kernels only: items[0] = number of chunks over all sequences,
                         // then from items[4] on, in launch order, four ints per chunk: sequence, chunk
                         // within it, first token row and length of the sequence
    int B, T, H;
    FastDiv dBH, dH;     // division by B * H and by H
};
struct SeqSpan { int64_t tok0; int len; };

// A read of a table that an EARLIER launch wrote and no workgroup of this one writes (cumulative lengths,
// chunk lists), at a wave-uniform address: through the constant address space, which makes it a scalar
// load whatever stores the kernel has issued before.  (As a plain global load inside a loop that also
// stores, it becomes a vector load whose arrival waits for every earlier load and store of the wave.)
__device__ __forceinline__ int load_table(const int* p) {
    return *(const __attribute__((address_space(4))) int*)p;
}
typedef int int4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ int4_t load_table4(const int* p) {      // p 16-byte aligned
    return *(const __attribute__((address_space(4))) int4_t*)p;
}

__device__ __forceinline__ SeqSpan seq_span(const SeqLayout& L, int bi) {
    if (L.cu == nullptr) return SeqSpan{(int64_t)bi * L.T, L.T};
    int s = load_table(L.cu + bi), e = load_table(L.cu + bi + 1);
    s = s < 0 ? 0 : (s > L.T ? L.T : s);
    e = e < s ? s : (e > L.T ? L.T : e);
    return SeqSpan{(int64_t)s, e - s};
}

// Sum over the eight lanes that share lane % 8 (lanes l, l ^ 8, l ^ 16, ..., i.e. one lane of every
// 8-lane group), delivered to all of them, without the LDS crossbar that __shfl_xor goes through: a DPP
// rotation inside the 16-lane rows, then gfx950's row and half swaps (v_permlane16_swap / v_permlane32_swap
// exchange the odd rows / the upper half of one register with the even rows / the lower half of the other,
// so with both registers equal to x the two results add up to x + x-of-the-neighbour).
__device__ __forceinline__ float sum_lane_groups_of_8(float x) {
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x128, 0xf, 0xf, true));   // row_ror:8
    const auto r16 = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(r16[0]) + __uint_as_float(r16[1]);
    const auto r32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r32[0]) + __uint_as_float(r32[1]);
}

// Maximum / sum of x over the four 16-lane rows of a wave (lanes l, l ^ 16, l ^ 32, l ^ 48), to all of them: the two
// swaps instead of two __shfl_xor, each of which is a trip through the LDS crossbar (72 cycles against 24).
__device__ __forceinline__ float max_over_rows(float x) {
    const auto r16 = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(r16[0]), __uint_as_float(r16[1]));
    const auto r32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r32[0]), __uint_as_float(r32[1]));
}
__device__ __forceinline__ float sum_over_rows(float x) {
    const auto r16 = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(r16[0]) + __uint_as_float(r16[1]);
    const auto r32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r32[0]) + __uint_as_float(r32[1]);
}

// Four values at once over the four 16-lane rows of a wave (lanes l, l + 16, l + 32, l + 48).  A swap of two
// DIFFERENT registers followed by one add halves two sums at a time: after v_permlane16_swap(a, b) the first
// register holds rows (a0, b0, a2, b2) and the second (a1, b1, a3, b3), so their sum holds a0 + a1 in row 0 and
// b0 + b1 in row 1; the same with c and d, then one v_permlane32_swap of the two sums and an add: row r of the
// result is the total of value r.  Three swaps and three adds where value by value takes eight swaps, eight moves
// and eight adds.
__device__ __forceinline__ float sum4_over_rows_scattered(float a, float b, float c, float d) {
    const auto s1 = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    const float ab = __uint_as_float(s1[0]) + __uint_as_float(s1[1]);
    const auto s2 = __builtin_amdgcn_permlane16_swap(__float_as_uint(c), __float_as_uint(d), false, false);
    const float cd = __uint_as_float(s2[0]) + __uint_as_float(s2[1]);
    const auto s3 = __builtin_amdgcn_permlane32_swap(__float_as_uint(ab), __float_as_uint(cd), false, false);
    return __uint_as_float(s3[0]) + __uint_as_float(s3[1]);
}
// ... and handed back to every row: rows (A, B, C, D) -> (A, B, A, B) and (C, D, C, D) -> A, B, C, D everywhere
__device__ __forceinline__ void sum4_over_rows(float& a, float& b, float& c, float& d) {
    const float t = sum4_over_rows_scattered(a, b, c, d);
    const auto g1 = __builtin_amdgcn_permlane32_swap(__float_as_uint(t), __float_as_uint(t), false, false);
    const auto g2 = __builtin_amdgcn_permlane16_swap(g1[0], g1[0], false, false);
    const auto g3 = __builtin_amdgcn_permlane16_swap(g1[1], g1[1], false, false);
    a = __uint_as_float(g2[0]); b = __uint_as_float(g2[1]); c = __uint_as_float(g3[0]); d = __uint_as_float(g3[1]);
}

// ---- N consecutive elements -> float --------------------------------------------
template <typename T> struct Io;

template <> struct Io<float> {
    static __device__ __forceinline__ void load4(const float* p, float (&x)[4]) {
        float4_t t = *reinterpret_cast<const float4_t*>(p);
        x[0] = t.x; x[1] = t.y; x[2] = t.z; x[3] = t.w;
    }
    static __device__ __forceinline__ void store4(float* p, const float (&x)[4]) {
        float4_t t = {x[0], x[1], x[2], x[3]};
        *reinterpret_cast<float4_t*>(p) = t;
    }
    static __device__ __forceinline__ float load1(const float* p) { return *p; }
    static __device__ __forceinline__ void store1(float* p, float x) { *p = x; }
};

template <> struct Io<bf16_t> {
    static __device__ __forceinline__ void load4(const bf16_t* p, float (&x)[4]) {
        u32x2_t t = *reinterpret_cast<const u32x2_t*>(p);
        x[0] = bf16_bits_to_f32(t.x & 0xffffu); x[1] = __uint_as_float(t.x & 0xffff0000u);
        x[2] = bf16_bits_to_f32(t.y & 0xffffu); x[3] = __uint_as_float(t.y & 0xffff0000u);
    }
    static __device__ __forceinline__ void store4(bf16_t* p, const float (&x)[4]) {
        bf16x4_t t = {(bf16_t)x[0], (bf16_t)x[1], (bf16_t)x[2], (bf16_t)x[3]};
        *reinterpret_cast<bf16x4_t*>(p) = t;
    }
    static __device__ __forceinline__ float load1(const bf16_t* p) { return (float)*p; }
    static __device__ __forceinline__ void store1(bf16_t* p, float x) { *p = (bf16_t)x; }
};

typedef _Float16 f16_t;
typedef _Float16 f16x4_t __attribute__((ext_vector_type(4)));

template <> struct Io<f16_t> {
    static __device__ __forceinline__ void load4(const f16_t* p, float (&x)[4]) {
        const f16x4_t t = *reinterpret_cast<const f16x4_t*>(p);
        x[0] = (float)t[0]; x[1] = (float)t[1]; x[2] = (float)t[2]; x[3] = (float)t[3];
    }
    static __device__ __forceinline__ void store4(f16_t* p, const float (&x)[4]) {
        f16x4_t t = {(f16_t)x[0], (f16_t)x[1], (f16_t)x[2], (f16_t)x[3]};
        *reinterpret_cast<f16x4_t*>(p) = t;
    }
    static __device__ __forceinline__ float load1(const f16_t* p) { return (float)*p; }
    static __device__ __forceinline__ void store1(f16_t* p, float x) { *p = (f16_t)x; }
};

template <typename T, int N>
__device__ __forceinline__ void load_n(const T* p, float (&x)[N]) {
    static_assert(N % 4 == 0, "multiples of 4");
#pragma unroll
    for (int i = 0; i < N; i += 4) {
        float t[4];
        Io<T>::load4(p + i, t);
        x[i] = t[0]; x[i + 1] = t[1]; x[i + 2] = t[2]; x[i + 3] = t[3];
    }
}

}  // namespace rwkv7
