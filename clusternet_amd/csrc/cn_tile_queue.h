// Tiles of a streaming kernel handed out through a counter in memory (device code only).
//
// A persistent grid that walks its tiles in a fixed pattern (grid-stride, or a range per workgroup) drifts apart:
// after a while the tiles in flight are spread over the whole tensor.  This part's memory rewards a stream that also
// writes for keeping the tiles in flight next to one another: measured on arithmetic-free kernels over 819.2 M
// elements, tiles drawn in order from a counter reach 6.9 TB/s for a copy against 6.0 TB/s grid-stride, 7.2 against
// 6.6 TB/s for pure writes, 6.7 against 6.3 TB/s for compression's pattern.  So the workgroups draw their tiles:
// whichever is free takes the next one, and the tiles in flight form one narrow window that advances through the
// tensor, as they do when the dispatcher starts a workgroup per tile.
//
// The counter must be 0 when the kernel starts and is left at 0: every workgroup draws until its ticket is past the
// last tile, so exactly gridDim.x tickets fail, and the workgroup that draws the last of them (ticket tiles +
// gridDim.x - 1) knows that nobody will draw again and clears the counter.  Kernels that share a counter must not
// overlap: the library keeps several and ties each to one launch stream (Context::tile_counter_for), whose order then is
// the order of the kernels on the counter; a launch that is being captured into a graph gets none and walks its tiles
// in a fixed pattern instead.
#pragma once

#include "cn_internal.h"

namespace cn {

struct TileQueue {
    uint32_t *counter;
    uint32_t tiles;
    uint32_t *slots;  // two words of LDS
    int turn;

    // Draws a ticket into the slot that next() will read after the coming barrier.  One lane draws; the ticket's
    // latency runs beside whatever the workgroup does until next().
    __device__ __forceinline__ void draw_ahead() {
        turn ^= 1;
        if (threadIdx.x == 0) {
            const uint32_t t = atomicAdd(counter, 1u);
            if (t == tiles + gridDim.x - 1u) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            slots[turn] = t;
        }
    }
    // The ticket drawn by the last draw_ahead(); contains a barrier.  A ticket >= tiles means: no tile left.
    __device__ __forceinline__ uint32_t next() {
        __syncthreads();
        return slots[turn];
    }
};

__device__ __forceinline__ TileQueue tile_queue(uint32_t *counter, uint32_t tiles, uint32_t *two_lds_words) {
    return TileQueue{counter, tiles, two_lds_words, 0};
}

// Calls tile_body(index of the tile's first 16-byte vector) for every tile of kTileVecs vectors.  kDrawn: a persistent
// grid draws the tiles from `counter` and waits for a tile's loads and stores before it takes the next (`slots`: two
// words of LDS); otherwise a grid-stride walk, which with as many workgroups as tiles is a workgroup per tile.
template <int kTileVecs, bool kDrawn, class F>
__device__ __forceinline__ void walk_tiles(size_t nvec, uint32_t *counter, uint32_t *slots, F &&tile_body) {
    const size_t tiles = (nvec + kTileVecs - 1) / kTileVecs;
    if (kDrawn) {
        TileQueue q = tile_queue(counter, (uint32_t)tiles, slots);
        q.draw_ahead();
        uint32_t tile = q.next();
        while (tile < tiles) {
            q.draw_ahead();
            tile_body((size_t)tile * kTileVecs);
            __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the tile's stores have been acknowledged
            tile = q.next();
        }
    } else {
        for (size_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) tile_body(tile * kTileVecs);
    }
}

// Element counts from which the streaming passes run as a persistent grid that draws its tiles (tensors beyond the
// 256 MB Infinity Cache); below it a workgroup per tile is faster (33.6 M elements: 64 us against 70 us).
constexpr size_t kDrawnFrom = (size_t)1 << 26;
// A drawn tile counts its tiles in 32 bits.
constexpr size_t kDrawnBelow = (size_t)1 << 40;

}  // namespace cn
