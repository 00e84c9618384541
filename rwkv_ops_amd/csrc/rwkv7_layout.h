// Where the chunks of the chunked kernels lie: sequences, chunk coordinates, workspace records.
#pragma once

#include "rwkv7_common.h"

namespace rwkv7 {

constexpr int CHUNK_TOKENS = 64;

// One chunk's place: which sequence and head, which chunk of it, where its tokens and its workspace
// record are.  Without cumulative lengths the launch index n = chunk * (B * H) + (b * H + h) is also the
// record's index: the heads of one chunk position are adjacent, so that concurrently running workgroups
// touch one contiguous region.  With them, launch index n = item * H + h, where the items list the chunks
// that exist, chunk position by chunk position; the records of sequence b start at (cu[b] / 64 + b) * H
// (a sequence has at most len / 64 + 1 chunks, so records of different sequences never overlap and
// (T / 64 + B) * H records hold them all, whatever the lengths are).
struct ChunkCoord {
    int64_t tok0;        // first token row of the sequence
    int64_t rec;         // index of the chunk's workspace record
    int bi, hi, c;       // sequence, head, chunk within the sequence
    int len, nt;         // tokens and chunks of the sequence
    bool live;           // false: the launch index is past the last chunk
};

__device__ __forceinline__ int64_t chunk_record(const SeqLayout& L, const SeqSpan& sp, int bi, int hi, int c) {
    return L.cu == nullptr ? ((int64_t)c * L.B + bi) * L.H + hi
                           : ((sp.tok0 >> 6) + bi + c) * L.H + hi;
}

// PACKED: 0 = the layout has no cumulative lengths, 1 = it has them, -1 = look (L.cu); kernels that are
// short of registers are compiled once for each case
template <int PACKED = -1>
__device__ __forceinline__ ChunkCoord chunk_coord(const SeqLayout& L, int n) {
    ChunkCoord q;
    if (PACKED == 0 || (PACKED < 0 && L.cu == nullptr)) {
        q.c = fast_div(n, L.dBH);
        const int bh = n - q.c * (L.B * L.H);
        q.bi = fast_div(bh, L.dH); q.hi = bh - q.bi * L.H;
        q.tok0 = (int64_t)q.bi * L.T; q.len = L.T; q.nt = (L.T + CHUNK_TOKENS - 1) / CHUNK_TOKENS;
        q.rec = n; q.live = true;
        return q;
    }
    const int item = fast_div(n, L.dH);
    q.hi = n - item * L.H;
    q.live = item < load_table(L.items);
    if (!q.live) { q.tok0 = 0; q.rec = 0; q.bi = 0; q.c = 0; q.len = 0; q.nt = 0; return q; }
    const int4_t e = load_table4(L.items + 4 + 4 * item);
    q.bi = e.x; q.c = e.y;
    const SeqSpan sp = SeqSpan{(int64_t)e.z, e.w};
    q.tok0 = sp.tok0; q.len = sp.len; q.nt = (sp.len + CHUNK_TOKENS - 1) / CHUNK_TOKENS;
    q.rec = chunk_record(L, sp, q.bi, q.hi, q.c);
    return q;
}

// The same for a kernel launched over a two- or three-dimensional grid, which spares the integer divisions:
// dense, grid (H, B, chunks): workgroup (x, y, z) = (head, sequence, chunk); packed, grid (H, items): (head, item).
// Workgroups are dispatched in the order of x + X (y + Y z), which is the launch index n of chunk_coord.  A
// one-dimensional grid (sizes beyond the 65535 that y and z can hold) falls back to chunk_coord.
__device__ __forceinline__ ChunkCoord chunk_coord_grid(const SeqLayout& L) {
    if (gridDim.y == 1 && gridDim.z == 1) return chunk_coord(L, (int)blockIdx.x);
    ChunkCoord q;
    q.hi = (int)blockIdx.x;
    if (L.cu == nullptr) {
        q.bi = (int)blockIdx.y; q.c = (int)blockIdx.z;
        q.tok0 = (int64_t)q.bi * L.T; q.len = L.T; q.nt = (L.T + CHUNK_TOKENS - 1) / CHUNK_TOKENS;
        q.rec = ((int64_t)q.c * L.B + q.bi) * L.H + q.hi; q.live = true;
        return q;
    }
    const int item = (int)blockIdx.y;
    q.live = item < load_table(L.items);
    if (!q.live) { q.tok0 = 0; q.rec = 0; q.bi = 0; q.c = 0; q.len = 0; q.nt = 0; return q; }
    const int4_t e = load_table4(L.items + 4 + 4 * item);
    q.bi = e.x; q.c = e.y;
    const SeqSpan sp = SeqSpan{(int64_t)e.z, e.w};
    q.tok0 = sp.tok0; q.len = sp.len; q.nt = (sp.len + CHUNK_TOKENS - 1) / CHUNK_TOKENS;
    q.rec = chunk_record(L, sp, q.bi, q.hi, q.c);
    return q;
}

// number of workspace records / upper bound of the number of chunks times H
__host__ __device__ inline int64_t chunk_records(int B, int T, int H, bool varlen) {
    return varlen ? ((int64_t)(T >> 6) + B) * H : (int64_t)B * H * ((T + CHUNK_TOKENS - 1) / CHUNK_TOKENS);
}

}  // namespace rwkv7
