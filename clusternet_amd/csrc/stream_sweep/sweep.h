// stream_sweep: what the memory system of one MI355X gives kernels that only move bytes, over a grid of access
// patterns, cache policies, tile shapes, occupancies and mappings of workgroups to addresses.  A measurement tool:
// nothing in libcnhip uses it.  It exists so that the throughput of compression_8bit / decompression_8bit /
// abs-max (source/basicOps.cu:1163-1176, 810-822 of the reference) can be read against ceilings that do not
// depend on how those kernels happen to be written.
//
// Kinds (bytes per element of the fp32 side): R4 read fp32; R4W1 read fp32, write one byte each (compression's
// pattern, 4-byte stores); R1W4 read bytes, write fp32 (decompression's, 4-byte loads); R4W4 copy; W4 write fp32;
// R4W1W / R1W4W the same as R4W1 / R1W4 with 16-byte accesses on the byte side.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <vector>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;

enum Kind { R4 = 0, R4W1 = 1, R1W4 = 2, R4W4 = 3, W4 = 4, R4W1W = 5, R1W4W = 6 };

// Cache-policy bits of the buffer instructions on gfx950: 1 = sc0, 2 = nt, 16 = sc1.
struct Variant {
    int kind, load_policy, store_policy, U, T;  // U 16-byte vectors per lane and tile, T lanes per workgroup
    void (*go)(unsigned grid, hipStream_t st, const void *in, void *out, uint32_t in_bytes, uint32_t out_bytes, uint32_t tiles,
               uint32_t chunk_tiles, int xcd_remap, int wait_for_stores, uint32_t *sink);
};

__device__ __forceinline__ rsrc_t make_rsrc(const void *p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, bytes, 0x00020000);
}

// Workgroup b owns the chunks b, b + G, b + 2G, ... of chunk_tiles consecutive tiles each: chunk_tiles 1 is a
// grid-stride walk, chunk_tiles = tiles / G one contiguous range per workgroup.  With xcd_remap the workgroups that
// one XCD receives (block ids congruent mod 8) own neighbouring chunks; xcd_remap 2 hands the chunks out through a
// ticket counter (sink[0]) instead, to whichever workgroup is free.
template <int KIND, int LAUX, int SAUX, int U, int T>
__global__ __launch_bounds__(T) void stream_kernel(const void *in, void *out, uint32_t in_bytes, uint32_t out_bytes, uint32_t tiles,
                                                   uint32_t chunk_tiles, int xcd_remap, int wait_for_stores, uint32_t *sink) {
    const uint32_t G = gridDim.x;
    uint32_t b = blockIdx.x;
    if (xcd_remap == 1) {
        const uint32_t xcd = b & 7u, idx = b >> 3, per = G >> 3, rem = G & 7u;
        b = xcd * per + (xcd < rem ? xcd : rem) + idx;
    }
    const rsrc_t rin = make_rsrc(in, in_bytes), rout = make_rsrc(out, out_bytes);
    const uint32_t tid = threadIdx.x;
    uint32_t running = 0;
    constexpr uint32_t kF = (uint32_t)T * U * 16u;  // bytes of a tile on the fp32 side
    constexpr uint32_t kC = (uint32_t)T * U * 4u;   // on the byte side
    // xcd_remap 2: the persistent workgroups take their tiles from a counter in memory, in the order in which they
    // become free (the next ticket is drawn before the current tile is processed, so its latency is hidden)
    __shared__ uint32_t ticket[2];
    const bool queue = xcd_remap == 2;
    uint32_t drawn = 0, turn = 0;
    if (queue) {
        if (tid == 0) ticket[0] = atomicAdd(sink, 1u);
        __syncthreads();
        drawn = ticket[0];
    }
    for (uint32_t chunk = queue ? drawn : b;; chunk = queue ? drawn : chunk + G) {
        const uint64_t first = (uint64_t)chunk * chunk_tiles;
        if (first >= tiles) break;
        uint32_t last = (uint32_t)first + chunk_tiles;
        if (last > tiles || last < (uint32_t)first) last = tiles;
        if (queue) {
            turn ^= 1u;
            if (tid == 0) ticket[turn] = atomicAdd(sink, 1u);
        }
        for (uint32_t t = (uint32_t)first; t < last; ++t) {
            const uint32_t tf = __builtin_amdgcn_readfirstlane(t * kF), tc = __builtin_amdgcn_readfirstlane(t * kC);
            if (KIND == R4 || KIND == R4W1 || KIND == R4W4 || KIND == R4W1W) {
                u32x4 v[U];
#pragma unroll
                for (int j = 0; j < U; ++j) v[j] = __builtin_amdgcn_raw_buffer_load_b128(rin, (j * T + tid) * 16u, tf, LAUX);
                if (KIND == R4) {
#pragma unroll
                    for (int j = 0; j < U; ++j) {
                        const uint32_t m = max(max(v[j].x, v[j].y), max(v[j].z, v[j].w));
                        running = m > running ? m : running;
                    }
                } else if (KIND == R4W1) {
#pragma unroll
                    for (int j = 0; j < U; ++j) {
                        const uint32_t p = (v[j].x >> 24) | ((v[j].y >> 24) << 8) | ((v[j].z >> 24) << 16) | ((v[j].w >> 24) << 24);
                        __builtin_amdgcn_raw_buffer_store_b32(p, rout, (j * T + tid) * 4u, tc, SAUX);
                    }
                } else if (KIND == R4W1W) {
#pragma unroll
                    for (int q = 0; q < U / 4; ++q) {
                        u32x4 p;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const u32x4 w = v[4 * q + e];
                            p[e] = (w.x >> 24) | ((w.y >> 24) << 8) | ((w.z >> 24) << 16) | ((w.w >> 24) << 24);
                        }
                        __builtin_amdgcn_raw_buffer_store_b128(p, rout, (q * T + tid) * 16u, tc, SAUX);
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < U; ++j) __builtin_amdgcn_raw_buffer_store_b128(v[j], rout, (j * T + tid) * 16u, tf, SAUX);
                }
            } else if (KIND == R1W4) {
                uint32_t w[U];
#pragma unroll
                for (int j = 0; j < U; ++j) w[j] = __builtin_amdgcn_raw_buffer_load_b32(rin, (j * T + tid) * 4u, tc, LAUX);
#pragma unroll
                for (int j = 0; j < U; ++j) {
                    const u32x4 o = {w[j] & 255u, (w[j] >> 8) & 255u, (w[j] >> 16) & 255u, w[j] >> 24};
                    __builtin_amdgcn_raw_buffer_store_b128(o, rout, (j * T + tid) * 16u, tf, SAUX);
                }
            } else if (KIND == R1W4W) {
                u32x4 w[U >= 4 ? U / 4 : 1];
#pragma unroll
                for (int q = 0; q < U / 4; ++q) w[q] = __builtin_amdgcn_raw_buffer_load_b128(rin, (q * T + tid) * 16u, tc, LAUX);
#pragma unroll
                for (int q = 0; q < U / 4; ++q)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t x = w[q][e];
                        const u32x4 o = {x & 255u, (x >> 8) & 255u, (x >> 16) & 255u, x >> 24};
                        __builtin_amdgcn_raw_buffer_store_b128(o, rout, ((4 * q + e) * T + tid) * 16u, tf, SAUX);
                    }
            } else {  // W4
                const u32x4 o = {tid, t, 0x3f800000u, b};
#pragma unroll
                for (int j = 0; j < U; ++j) __builtin_amdgcn_raw_buffer_store_b128(o, rout, (j * T + tid) * 16u, tf, SAUX);
            }
            // closed loop: nothing of the next tile is requested before this tile's stores have been acknowledged
            if (KIND != R4 && wait_for_stores) __builtin_amdgcn_s_waitcnt(0x0f70);
        }
        if (queue) {
            __syncthreads();
            drawn = ticket[turn];
        }
    }
    // the maximum must be wanted by something; no input holds this pattern, so nothing is ever stored
    if (KIND == R4 && running == 0xffffffffu) sink[tid] = running;
}

template <int KIND, int LAUX, int SAUX, int U, int T>
static void go(unsigned grid, hipStream_t st, const void *in, void *out, uint32_t ib, uint32_t ob, uint32_t tiles, uint32_t chunk,
               int remap, int wait, uint32_t *sink) {
    if (remap == 2) (void)hipMemsetAsync(sink, 0, 4, st);  // the ticket counter
    hipLaunchKernelGGL((stream_kernel<KIND, LAUX, SAUX, U, T>), dim3(grid), dim3(T), 0, st, in, out, ib, ob, tiles, chunk, remap,
                       wait, sink);
}

// One translation unit per kind (compiled with -DSWEEP_KIND=k) registers that kind's variants.
void register_kind_0(std::vector<Variant> &);
void register_kind_1(std::vector<Variant> &);
void register_kind_2(std::vector<Variant> &);
void register_kind_3(std::vector<Variant> &);
void register_kind_4(std::vector<Variant> &);
void register_kind_5(std::vector<Variant> &);
void register_kind_6(std::vector<Variant> &);
