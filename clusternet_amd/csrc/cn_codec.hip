// 8-bit codec and abs-max kernels for gfx950.  All three are HBM-bound streaming kernels:
//   compress    4 B read + 1 B written per element
//   decompress  1 B read + 4 B written per element
//   absmax      4 B read per element
// Each lane moves 16-byte vectors laid out so that one wavefront instruction touches one
// contiguous 1 KiB (fp32 side) / 256 B (code side) span.
//
// What a stream that also writes reaches on this part depends sharply on the window of addresses in flight.
// Decompression (mostly writes) runs a workgroup per 4096-element tile, as many workgroups as tiles, so that the
// dispatcher keeps the tiles in flight next to one another: 6.9 TB/s, against 6.1 TB/s for the best persistent grid.
// Compression cannot start a workgroup per tile (a workgroup first needs its encoder table in LDS: 40 KB copied, or
// built in 9 000 cycles); large tensors take compress_stream_kernel, one persistent workgroup per compute unit that
// draws its tiles in order from a counter, which keeps the same narrow window (6.6 TB/s, against 6.4 TB/s on a
// grid-stride walk), addressed through a buffer descriptor per tile (a uniform base and a 32-bit lane offset; the
// descriptor's range replaces the bounds test of the last tile), read and written with the non-temporal hint.
//
// Three encoders give the same codes (compress_impl picks by size): the literal procedure element by element, the
// fixed table on the quotient x / precision (cn_xlut.h, cn_encode_table.h) and the table built per call for the
// call's precision (cn_encode_table.h).
#include <type_traits>

#include "cn_internal.h"
#include "cn_xlut.h"
#include "cn_encode_table.h"
#include "cn_tile_queue.h"

namespace cn {

constexpr int kThreads = 256;
constexpr int kVecPerThread = 4;                         // float4 per lane per tile
constexpr int kTileVec = kThreads * kVecPerThread;       // float4 per workgroup tile (4096 floats)

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// kUpdate: besides the codes, y += alpha * (decoded value of each code), as decompress_axpy would add it
// afterwards: the gradient's codes for the exchange and the own weight update in one pass over both arrays.
template <bool kVector, bool kUpdate, bool kQuotient = false>
__global__ __launch_bounds__(kThreads) void compress_kernel(
    const float *__restrict__ x, float precision_value, const float *__restrict__ precision_ptr,
    size_t n, uint8_t *__restrict__ codes, const XStep *__restrict__ steps, int step_count,
    const float *__restrict__ table, float alpha, float *__restrict__ y, const XEntry *__restrict__ quotient_table = nullptr) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    EncodeShared &sh = *reinterpret_cast<EncodeShared *>(smem_raw);
    float *dlut = reinterpret_cast<float *>(smem_raw + sizeof(EncodeShared));  // kUpdate: decode table times alpha
    const float precision = precision_ptr ? *precision_ptr : precision_value;

    // The workgroup's first tile is requested before the table is built, so that its memory latency runs
    // beside those of the table's inputs: a small input is one or two tiles per workgroup.
    const size_t nvec = n / 4;
    const f32x4 *x4 = reinterpret_cast<const f32x4 *>(x);
    f32x4 *y4 = reinterpret_cast<f32x4 *>(y);
    const size_t tiles = (nvec + kTileVec - 1) / kTileVec;
    auto load_tile = [&](size_t tile, f32x4 (&v)[kVecPerThread], f32x4 (&w)[kVecPerThread]) {
        const size_t base = tile * kTileVec + threadIdx.x;
#pragma unroll
        for (int j = 0; j < kVecPerThread; ++j) {
            size_t i = base + (size_t)j * kThreads;
            v[j] = (i < nvec) ? __builtin_nontemporal_load(&x4[i]) : f32x4{0.f, 0.f, 0.f, 0.f};
            if (kUpdate) w[j] = (i < nvec) ? __builtin_nontemporal_load(&y4[i]) : f32x4{0.f, 0.f, 0.f, 0.f};
        }
    };
    // Two register sets: the loads of the next tile are in flight while this one is encoded,
    // so the memory pipe stays busy even with only a few wavefronts per SIMD.
    f32x4 va[kVecPerThread], vb[kVecPerThread], wa[kUpdate ? kVecPerThread : 1], wb[kUpdate ? kVecPerThread : 1];
    auto load = [&](size_t tile, f32x4 (&v)[kVecPerThread], f32x4 (&w)[kUpdate ? kVecPerThread : 1]) {
        load_tile(tile, v, reinterpret_cast<f32x4 (&)[kVecPerThread]>(w));
    };
    QuotientTableCopy<kThreads> copy;
    if (kQuotient) copy.request(quotient_table);  // ahead of the tile: loads return in order
    if (kVector && blockIdx.x < tiles) load(blockIdx.x, va, wa);

    bool exact_only = false;
    if (kQuotient) {
        copy.store(sh.lut);
        if (!kUpdate) __syncthreads();
    } else {
        exact_only = !build_table(sh, steps, step_count, precision, table);
    }
    const double scale = quotient_scale(precision);
    const uint32_t first_of_one = xlut_first(1.0f);
    if (kUpdate) {
        const int t = threadIdx.x;
        if (t < 126) {
            const float v = table[t] * precision;
            dlut[t] = alpha * v;
            dlut[t + 128] = alpha * (-v);
        } else if (t == 126) {
            dlut[126] = alpha * precision;
            dlut[127] = alpha * precision;
            dlut[254] = alpha * precision;
            dlut[255] = alpha * (-precision);
        }
        __syncthreads();
    }
    const uint32_t first = xlut_first(precision);
    auto encode = [&](float v) -> uint32_t {
        const uint32_t bits = __float_as_uint(v);
        if (kQuotient) return encode_by_quotient(bits, scale, sh.lut, first_of_one);
        return xlut_code(bits, sh.lut[xlut_index(bits & 0x7fffffffu, first)]);
    };

    if (kVector) {
        uint32_t *c4 = reinterpret_cast<uint32_t *>(codes);
        auto encode_tile = [&](size_t tile, const f32x4 (&v)[kVecPerThread], f32x4 (&w)[kVecPerThread]) {
            const size_t base = tile * kTileVec + threadIdx.x;
            uint32_t packed[kVecPerThread];
            if (!exact_only) {
#pragma unroll
                for (int j = 0; j < kVecPerThread; ++j)
                    packed[j] = encode(v[j].x) | (encode(v[j].y) << 8) | (encode(v[j].z) << 16) | (encode(v[j].w) << 24);
            } else {
#pragma unroll
                for (int j = 0; j < kVecPerThread; ++j)
                    packed[j] = encode_exact(v[j].x, precision, sh.slot) | (encode_exact(v[j].y, precision, sh.slot) << 8) |
                                (encode_exact(v[j].z, precision, sh.slot) << 16) |
                                (encode_exact(v[j].w, precision, sh.slot) << 24);
            }
#pragma unroll
            for (int j = 0; j < kVecPerThread; ++j) {
                size_t i = base + (size_t)j * kThreads;
                if (i < nvec) __builtin_nontemporal_store(packed[j], &c4[i]);
                if (kUpdate) {
                    f32x4 o;
                    o.x = w[j].x + dlut[packed[j] & 0xffu];
                    o.y = w[j].y + dlut[(packed[j] >> 8) & 0xffu];
                    o.z = w[j].z + dlut[(packed[j] >> 16) & 0xffu];
                    o.w = w[j].w + dlut[packed[j] >> 24];
                    if (i < nvec) __builtin_nontemporal_store(o, &y4[i]);
                }
            }
        };
        auto finish = [&](size_t tile, const f32x4 (&v)[kVecPerThread], f32x4 (&w)[kUpdate ? kVecPerThread : 1]) {
            encode_tile(tile, v, reinterpret_cast<f32x4 (&)[kVecPerThread]>(w));
        };
        size_t t0 = blockIdx.x;
        if (t0 < tiles) {  // its loads are on their way since before the table
            for (;;) {
                const size_t t1 = t0 + gridDim.x;
                if (t1 < tiles) load(t1, vb, wb);
                finish(t0, va, wa);
                if (t1 >= tiles) break;
                t0 = t1 + gridDim.x;
                if (t0 < tiles) load(t0, va, wa);
                finish(t1, vb, wb);
                if (t0 >= tiles) break;
            }
        }
        // ragged tail (n % 4 elements)
        if (blockIdx.x == 0) {
            size_t i = nvec * 4 + threadIdx.x;
            if (i < n) {
                const uint32_t c = exact_only ? encode_exact(x[i], precision, sh.slot) : encode(x[i]);
                codes[i] = (uint8_t)c;
                if (kUpdate) y[i] = y[i] + dlut[c];
            }
        }
    } else {
        for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (size_t)gridDim.x * kThreads) {
            const uint32_t c = exact_only ? encode_exact(x[i], precision, sh.slot) : encode(x[i]);
            codes[i] = (uint8_t)c;
            if (kUpdate) y[i] = y[i] + dlut[c];
        }
    }
}

// ---- the literal procedure for small tensors ---------------------------------------------------------------
// A workgroup's table is 40 KB to copy, or about 9 000 cycles to build, before the first element is encoded; the
// literal procedure (division and pivot search, encode_exact) costs about 70 instructions per element and needs only
// the 126-entry codebook.  A tensor of up to a few hundred thousand elements spread over the whole chip is a handful
// of elements per lane, which the literal procedure finishes before a table would be there.  Four elements per lane
// and step, evaluated level by level so that the search's LDS reads overlap; same bits as the tables by construction
// (they are made of evaluations of this procedure).
template <bool kVector, bool kUpdate>
__global__ __launch_bounds__(kThreads) void compress_literal_kernel(
    const float *__restrict__ x, float precision_value, const float *__restrict__ precision_ptr, size_t n,
    uint8_t *__restrict__ codes, const float *__restrict__ table, float alpha, float *__restrict__ y) {
    __shared__ float slot[128];
    __shared__ float dlut[kUpdate ? 256 : 1];
    const int t = threadIdx.x;
    const float precision = precision_ptr ? *precision_ptr : precision_value;
    const size_t nvec = kVector ? n / 4 : 0;
    const size_t v0 = (size_t)blockIdx.x * kThreads + t;
    f32x4 first{0.f, 0.f, 0.f, 0.f};
    if (kVector && v0 < nvec) first = reinterpret_cast<const f32x4 *>(x)[v0];  // beside the codebook's latency
    if (t < 126) {
        const float c = table[t];
        slot[t] = c;
        if (kUpdate) {
            const float v = c * precision;
            dlut[t] = alpha * v;
            dlut[t + 128] = alpha * (-v);
        }
    } else if (t == 126) {
        slot[126] = 1.0f;
        slot[127] = 0.0f;
        if (kUpdate) {
            dlut[126] = alpha * precision;
            dlut[127] = alpha * precision;
            dlut[254] = alpha * precision;
            dlut[255] = alpha * (-precision);
        }
    }
    __syncthreads();
    if (kVector) {
        for (size_t v = v0; v < nvec; v += (size_t)gridDim.x * kThreads) {
            const f32x4 in = (v == v0) ? first : reinterpret_cast<const f32x4 *>(x)[v];
            const uint32_t bits[4] = {__float_as_uint(in.x), __float_as_uint(in.y), __float_as_uint(in.z), __float_as_uint(in.w)};
            uint32_t c[4];
            encode_exact_many<4>(bits, precision, slot, c);
            reinterpret_cast<uint32_t *>(codes)[v] = c[0] | (c[1] << 8) | (c[2] << 16) | (c[3] << 24);
            if (kUpdate) {
                f32x4 w = reinterpret_cast<f32x4 *>(y)[v];
                w.x = w.x + dlut[c[0]];
                w.y = w.y + dlut[c[1]];
                w.z = w.z + dlut[c[2]];
                w.w = w.w + dlut[c[3]];
                reinterpret_cast<f32x4 *>(y)[v] = w;
            }
        }
    }
    // without vectors: everything; with them: the n % 4 elements behind the last whole vector
    for (size_t i = nvec * 4 + (size_t)blockIdx.x * kThreads + t; i < n; i += (size_t)gridDim.x * kThreads) {
        const uint32_t c = encode_exact(x[i], precision, slot);
        codes[i] = (uint8_t)c;
        if (kUpdate) y[i] = y[i] + dlut[c];
    }
}

// ---- streaming forms for large tensors ---------------------------------------------------------------------
typedef __amdgpu_buffer_rsrc_t rsrc_t;
constexpr int kAuxNt = 2;            // cache policy bits of the buffer instructions: nt
constexpr int kAuxSc0Sc1Nt = 19;     // sc0 sc1 nt
__device__ __forceinline__ rsrc_t tile_rsrc(const void *base, uint32_t bytes) {
    // 0x00020000: 32-bit untyped data; accesses at or beyond `bytes` read zero and write nothing
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes, 0x00020000);
}

// Compression of whole float4 groups: a tile is T * U float4, all of its loads are issued at once and awaited
// together, then encoded and stored; the next tile's loads go out right behind the stores.  Two shapes: 1024 x 12
// (192 KiB of input per tile), one workgroup per compute unit, tiles drawn in order from a counter (`queue`,
// cn_tile_queue.h) for tensors that stream from HBM; 512 x 10 with two workgroups per compute unit on a grid-stride
// walk (`queue` NULL) below that.  kQuotient: the table on the quotient, copied from `quotient_table`, instead of a
// table built for the precision.
template <int T, int U, bool kUpdate, bool kQuotient = false>
__global__ __launch_bounds__(T) void compress_stream_kernel(
    const float *__restrict__ x, float precision_value, const float *__restrict__ precision_ptr, size_t n,
    uint8_t *__restrict__ codes, const XStep *__restrict__ steps, int step_count, const float *__restrict__ table,
    uint32_t *__restrict__ queue, float alpha, float *__restrict__ y, const XEntry *__restrict__ quotient_table = nullptr) {
    constexpr uint32_t kVecs = T * U;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    EncodeShared &sh = *reinterpret_cast<EncodeShared *>(smem_raw);
    float *dlut = reinterpret_cast<float *>(smem_raw + sizeof(EncodeShared));  // kUpdate: decode table times alpha
    __shared__ uint32_t queue_slots[2];
    const float precision = precision_ptr ? *precision_ptr : precision_value;
    const size_t nvec = n / 4;
    const size_t tiles = (nvec + kVecs - 1) / kVecs;
    const uint32_t tid = threadIdx.x;
    u32x4 v[U], w[kUpdate ? U : 1];
    auto load = [&](size_t tile) {
        const size_t left = nvec - tile * kVecs;
        const uint32_t bytes = (uint32_t)(left < kVecs ? left : kVecs) * 16u;
        const rsrc_t r = tile_rsrc(x + tile * (size_t)kVecs * 4, bytes);
#pragma unroll
        for (int j = 0; j < U; ++j) v[j] = __builtin_amdgcn_raw_buffer_load_b128(r, (j * T + tid) * 16u, 0, kAuxNt);
        if (kUpdate) {
            const rsrc_t ry = tile_rsrc(y + tile * (size_t)kVecs * 4, bytes);
#pragma unroll
            for (int j = 0; j < U; ++j) w[j] = __builtin_amdgcn_raw_buffer_load_b128(ry, (j * T + tid) * 16u, 0, kAuxNt);
        }
    };
    // tiles are drawn from a counter (cn_tile_queue.h); without one, a grid-stride walk
    TileQueue q = tile_queue(queue, (uint32_t)tiles, queue_slots);
    size_t tile = blockIdx.x;
    QuotientTableCopy<T> copy;
    if (kQuotient) copy.request(quotient_table);  // ahead of the tile: loads return in order
    if (queue) {
        q.draw_ahead();
        tile = q.next();
    }
    if (tile < tiles) {
        load(tile);  // on their way while the table is built
        if (queue) q.draw_ahead();
    }
    bool exact_only = false;
    if (kQuotient) {
        copy.store(sh.lut);
        if (!kUpdate) __syncthreads();
    } else {
        exact_only = !build_table(sh, steps, step_count, precision, table);
    }
    const double scale = quotient_scale(precision);
    const uint32_t first_of_one = xlut_first(1.0f);
    if (kUpdate) {
        if (tid < 126) {
            const float d = table[tid] * precision;
            dlut[tid] = alpha * d;
            dlut[tid + 128] = alpha * (-d);
        } else if (tid == 126) {
            dlut[126] = alpha * precision;
            dlut[127] = alpha * precision;
            dlut[254] = alpha * precision;
            dlut[255] = alpha * (-precision);
        }
        __syncthreads();
    }
    const uint32_t first = xlut_first(precision);
    // `exact` is a type: the table look-up, or (where no table can be trusted) the literal procedure per element
    auto run = [&](auto exact) {
        auto encode = [&](uint32_t bits) -> uint32_t {
            if (kQuotient) return encode_by_quotient(bits, scale, sh.lut, first_of_one);
            if (decltype(exact)::value) return encode_exact(__uint_as_float(bits), precision, sh.slot);
            return xlut_code(bits, sh.lut[xlut_index(bits & 0x7fffffffu, first)]);
        };
        while (tile < tiles) {
            const size_t left = nvec - tile * kVecs;
            const uint32_t vecs = (uint32_t)(left < kVecs ? left : kVecs);
            const rsrc_t r = tile_rsrc(codes + tile * (size_t)kVecs * 4, vecs * 4u);
            uint32_t packed[U];
            // the whole tile has arrived before the first element is encoded: while a wavefront encodes it has
            // nothing in flight, which is what keeps the bytes in flight per compute unit at the optimum
            __builtin_amdgcn_s_waitcnt(0x0f70);
#pragma unroll
            for (int j = 0; j < U; ++j)
                packed[j] = encode(v[j].x) | (encode(v[j].y) << 8) | (encode(v[j].z) << 16) | (encode(v[j].w) << 24);
#pragma unroll
            for (int j = 0; j < U; ++j) __builtin_amdgcn_raw_buffer_store_b32(packed[j], r, (j * T + tid) * 4u, 0, kAuxNt);
            if (kUpdate) {
                const rsrc_t ry = tile_rsrc(y + tile * (size_t)kVecs * 4, vecs * 16u);
#pragma unroll
                for (int j = 0; j < U; ++j) {
                    u32x4 o;
                    o.x = __float_as_uint(__uint_as_float(w[j].x) + dlut[packed[j] & 0xffu]);
                    o.y = __float_as_uint(__uint_as_float(w[j].y) + dlut[(packed[j] >> 8) & 0xffu]);
                    o.z = __float_as_uint(__uint_as_float(w[j].z) + dlut[(packed[j] >> 16) & 0xffu]);
                    o.w = __float_as_uint(__uint_as_float(w[j].w) + dlut[packed[j] >> 24]);
                    __builtin_amdgcn_raw_buffer_store_b128(o, ry, (j * T + tid) * 16u, 0, kAuxNt);
                }
            }
            tile = queue ? (size_t)q.next() : tile + gridDim.x;
            if (tile < tiles) {
                load(tile);
                if (queue) q.draw_ahead();
            }
        }
        if (blockIdx.x == 0) {  // ragged tail (n % 4 elements)
            const size_t i = nvec * 4 + tid;
            if (i < n) {
                const uint32_t c = encode(__float_as_uint(x[i]));
                codes[i] = (uint8_t)c;
                if (kUpdate) y[i] = y[i] + dlut[c];
            }
        }
    };
    if (exact_only) run(std::true_type{}); else run(std::false_type{});
}

// Decompression with a workgroup per tile and as many workgroups as tiles, placed by the dispatcher as compute
// units free up: the workgroups in flight at any moment then cover one narrow, advancing window of addresses, which
// is what this part's memory rewards in a stream that mostly writes (measured on arithmetic-free kernels: 6.6 TB/s
// for 1 byte read + 4 written this way, 6.2 TB/s for the best persistent grid).  The price is a decode table per
// 2048 elements: its inputs are requested together with the tile's codes, so it costs a barrier, not a latency.
template <int T, int U>
__global__ __launch_bounds__(T) void decompress_tile_kernel(
    const uint8_t *__restrict__ codes, float precision_value, const float *__restrict__ precision_ptr, size_t n,
    float *__restrict__ out, const float *__restrict__ table, const float *__restrict__ given_lut) {
    static_assert(T >= 256, "one lane per table entry");
    constexpr uint32_t kVecs = T * U;
    __shared__ float lut[256];
    const uint32_t tid = threadIdx.x;
    const size_t nvec = n / 4;
    const size_t first = (size_t)blockIdx.x * kVecs;
    const size_t left = first < nvec ? nvec - first : 0;
    const uint32_t vecs = (uint32_t)(left < kVecs ? left : kVecs);
    const rsrc_t rc = tile_rsrc(codes + first * 4, vecs * 4u);
    const rsrc_t ro = tile_rsrc(out + first * 4, vecs * 16u);
    uint32_t w[U];
#pragma unroll
    for (int j = 0; j < U; ++j) w[j] = __builtin_amdgcn_raw_buffer_load_b32(rc, (j * T + tid) * 4u, 0, 0);
    const float precision = precision_ptr ? *precision_ptr : precision_value;
    if (given_lut) {  // the caller's own 256-entry table instead of the codec's
        if (tid < 256) lut[tid] = given_lut[tid];
    } else if (tid < 126) {
        const float v = table[tid] * precision;
        lut[tid] = v;
        lut[tid + 128] = -v;
    } else if (tid == 126) {
        lut[126] = precision;
        lut[127] = precision;
        lut[254] = precision;
        lut[255] = -precision;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < U; ++j) {
        u32x4 o;
        o.x = __float_as_uint(lut[w[j] & 0xffu]);
        o.y = __float_as_uint(lut[(w[j] >> 8) & 0xffu]);
        o.z = __float_as_uint(lut[(w[j] >> 16) & 0xffu]);
        o.w = __float_as_uint(lut[w[j] >> 24]);
        __builtin_amdgcn_raw_buffer_store_b128(o, ro, (j * T + tid) * 16u, 0, kAuxSc0Sc1Nt);
    }
    if (blockIdx.x == 0) {  // the n % 4 elements behind the last whole word
        const size_t i = nvec * 4 + tid;
        if (i < n) out[i] = lut[codes[i]];
    }
}

// Follows kDecompression_8bit (source/clusterKernels.cu:1135-1160): a 256-entry table scaled by
// the precision, rebuilt once per workgroup, then a pure gather.  Element by element, for buffers that are not
// aligned to whole words; aligned ones take decompress_tile_kernel.
__global__ __launch_bounds__(kThreads) void decompress_kernel(
    const uint8_t *__restrict__ codes, float precision_value, const float *__restrict__ precision_ptr,
    size_t n, float *__restrict__ out, const float *__restrict__ table, const float *__restrict__ given_lut) {
    __shared__ float lut[256];
    const float precision = precision_ptr ? *precision_ptr : precision_value;
    if (given_lut) {  // the caller's own 256-entry table instead of the codec's
        lut[threadIdx.x] = given_lut[threadIdx.x];
    } else if (threadIdx.x < 126) {
        float v = table[threadIdx.x] * precision;
        lut[threadIdx.x] = v;
        lut[threadIdx.x + 128] = -v;
    } else if (threadIdx.x == 126) {
        lut[126] = precision;
        lut[127] = precision;
        lut[254] = precision;
        lut[255] = -precision;
    }
    __syncthreads();
    for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (size_t)gridDim.x * kThreads)
        out[i] = lut[codes[i]];
}

// ---- abs-max ------------------------------------------------------------------------------------
// Non-negative fp32 values order like their bit patterns, so the reduction runs on
// (pattern & 0x7fffffff) with integer max: exact, order-independent, and a NaN (pattern above
// 0x7f800000) wins and is returned as NaN.
__device__ __forceinline__ uint32_t wave_max(uint32_t v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = max(v, (uint32_t)__shfl_xor((int)v, off, 64));
    return v;
}

__device__ __forceinline__ uint32_t block_max(uint32_t v, uint32_t *smem) {
    v = wave_max(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    if (wave == 0) {
        v = (lane < (int)(blockDim.x >> 6)) ? smem[lane] : 0u;
        v = wave_max(v);
    }
    return v;  // valid in wave 0
}

// kAbs: key = |x| pattern.  Otherwise (plain max, start value -1 as in the reference's reduction)
// the key is the usual order-preserving map of a signed fp32 pattern onto unsigned integers.
template <bool kAbs>
__device__ __forceinline__ uint32_t max_key(uint32_t bits) {
    if (kAbs) return bits & 0x7fffffffu;
    return (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
}
template <bool kAbs>
__device__ __forceinline__ float max_unkey(uint32_t key) {
    if (kAbs) return __uint_as_float(key);
    return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}

// One arrival at a ticket line: the 64-bit word at `line` holds the running maximum in its low half and the number of
// arrivals in its high half.  The maximum is folded in with a 32-bit atomicMax on the low half, the arrival counted
// with a 64-bit atomicAdd of 1 << 32 on the whole word, which leaves the low half as it is and returns both halves as
// they were: whoever finds members - 1 earlier arrivals holds, in the low half of what its own count returned, the
// maximum over all members (each member's fold comes before its count in the order of operations on that word, and
// all the counts came before this one), without a further read.  Both atomics return a value and the count's
// operand is made to depend on what the fold returned, so the fold has been performed before the count is issued;
// `fenced` puts a release fence between the two and an acquire fence behind the count, the memory model's own form
// for a pair of locations.  Returns true for the last arrival, with *all = the maximum; it then puts the word back to 0.
__device__ __forceinline__ bool ticket_arrive(uint32_t *line, uint32_t value, uint32_t members, int fenced, uint32_t *all) {
    const uint32_t before = atomicMax(line, value);
    unsigned long long one = 1ull << 32;
    asm volatile("" : "+v"(one) : "v"(before));  // `one` is not available before `before` is
    if (fenced) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    const unsigned long long seen = atomicAdd(reinterpret_cast<unsigned long long *>(line), one);
    if ((uint32_t)(seen >> 32) != members - 1) return false;
    if (fenced) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    __hip_atomic_store(reinterpret_cast<unsigned long long *>(line), 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *all = (uint32_t)seen;  // includes `value`: this lane's fold was performed before its count
    return true;
}

template <bool kVector, bool kAbs>
__global__ __launch_bounds__(kThreads) void absmax_kernel(const float *__restrict__ x, size_t n,
                                                          float *__restrict__ out,
                                                          uint32_t *__restrict__ tickets, int fenced) {
    __shared__ uint32_t smem[kThreads / 64];
    const uint32_t start = kAbs ? 0u : max_key<false>(0xbf800000u);
    uint32_t m = start;
    if (kVector) {
        const size_t nvec = n / 4;
        const u32x4 *x4 = reinterpret_cast<const u32x4 *>(x);
        const size_t tiles = (nvec + kTileVec - 1) / kTileVec;
        for (size_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
            const size_t base = tile * kTileVec + threadIdx.x;
            u32x4 v[kVecPerThread];
#pragma unroll
            for (int j = 0; j < kVecPerThread; ++j) {
                size_t i = base + (size_t)j * kThreads;
                // positions past the end take the pattern whose key is the smallest possible
                const uint32_t pad = kAbs ? 0u : 0xffffffffu;
                v[j] = (i < nvec) ? __builtin_nontemporal_load(&x4[i]) : u32x4{pad, pad, pad, pad};
            }
#pragma unroll
            for (int j = 0; j < kVecPerThread; ++j) {
                m = max(m, max_key<kAbs>(v[j].x));
                m = max(m, max_key<kAbs>(v[j].y));
                m = max(m, max_key<kAbs>(v[j].z));
                m = max(m, max_key<kAbs>(v[j].w));
            }
        }
        if (blockIdx.x == 0) {
            size_t i = nvec * 4 + threadIdx.x;
            if (i < n) m = max(m, max_key<kAbs>(__float_as_uint(x[i])));
        }
    } else {
        for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (size_t)gridDim.x * kThreads)
            m = max(m, max_key<kAbs>(__float_as_uint(x[i])));
    }
    m = block_max(m, smem);
    // Two-level ticket (ticket_arrive): the workgroup arrives at the line of its group of eight; the last of a group
    // carries the group's maximum to the line of the groups, and the last group writes the result.  Atomics on one
    // word are performed one after the other, about 12 ns each, hence the groups: their words lie on lines of their
    // own.  Ordering by data dependence instead of by fences costs far less here (a release fence per workgroup
    // writes the L2 back; nothing in this kernel needs that) and rests on a property of this part: a returning
    // atomic has been performed at the device's coherence point before an instruction that consumes its result
    // issues.  `fenced` (cn_host_reduction_fences) switches to the memory model's own form; the tests hold the two
    // forms to the same bits.  A grid of one workgroup, or of one group, skips what it does not need.
    if (threadIdx.x == 0) {
        const uint32_t groups = (gridDim.x + kTicketGroup - 1) / kTicketGroup;
        const uint32_t group = blockIdx.x / kTicketGroup;
        const uint32_t left = gridDim.x - group * kTicketGroup;
        const uint32_t members = left < (uint32_t)kTicketGroup ? left : (uint32_t)kTicketGroup;
        uint32_t all = m;
        if (gridDim.x == 1) {
            out[0] = max_unkey<kAbs>(all);
        } else if (ticket_arrive(tickets + (1 + group) * kTicketStride, m, members, fenced, &all)) {
            if (groups == 1 || ticket_arrive(tickets, all, groups, fenced, &all)) out[0] = max_unkey<kAbs>(all);
        }
    }
}

// ---- abs-max and compression in one launch ------------------------------------------------------------------
// Phase 1: every workgroup folds the maximum of its tiles into the two-level ticket of absmax_kernel (same words,
// same ordering; kernels of one stream do not overlap).  Whoever arrives last of all holds the maximum and
// publishes it, together with the number of this call, in a word of every group's line; every workgroup waits
// for that word on its own group's line (eight readers per line) and goes on to phase 2: the codes of the same
// tiles under that maximum (the encoder's table is the one on the quotient, which does not depend on the precision
// and is copied into LDS before the first phase), whose second read comes from the caches for tensors they can hold.
// The grid is sized to be resident as a whole, so the wait ends; it is bounded all the same: a workgroup that
// gives up (part of the grid not resident because another kernel holds compute units) takes the maximum over the
// whole tensor by itself, slow and still exact, and every workgroup ends either way.
// The number of the call is read from device memory at the start (tickets[kCallWord]) and advanced by the last
// arriver, after everyone has read it: a captured launch replays correctly, and nothing has to be reset.
constexpr int kCallWord = 8;    // in the top line: number of the last completed call
constexpr int kResultWord = 8;  // in a group's line (64-bit): call number << 32 | maximum

__global__ __launch_bounds__(kThreads) void absmax_compress_kernel(
    const float *__restrict__ x, size_t n, uint8_t *__restrict__ codes, float *__restrict__ precision_out,
    uint32_t *__restrict__ tickets, uint32_t spin_limit, const XEntry *__restrict__ quotient_table, int fenced) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    XEntry *lut = reinterpret_cast<XEntry *>(smem_raw);  // kXEntries entries
    QuotientTableCopy<kThreads> copy;
    copy.request(quotient_table);  // ahead of the tiles: loads return in order
    __shared__ uint32_t red[kThreads / 64];
    __shared__ uint32_t s_key, s_complete;
    const size_t nvec = n / 4;
    const u32x4 *x4 = reinterpret_cast<const u32x4 *>(x);
    const size_t tiles = (nvec + kTileVec - 1) / kTileVec;
    const uint32_t groups = (gridDim.x + kTicketGroup - 1) / kTicketGroup;
    const uint32_t group = blockIdx.x / kTicketGroup;
    uint32_t call = 0;
    if (threadIdx.x == 0) call = __hip_atomic_load(&tickets[kCallWord], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;
    // maximum over the tiles first, first + stride, ...; the ragged tail belongs to whoever takes tile 0
    auto fold = [](uint32_t m, const u32x4 (&v)[kVecPerThread]) -> uint32_t {
#pragma unroll
        for (int j = 0; j < kVecPerThread; ++j)
            m = max(max(m, v[j].x & 0x7fffffffu), max(max(v[j].y & 0x7fffffffu, v[j].z & 0x7fffffffu), v[j].w & 0x7fffffffu));
        return m;
    };
    auto load_tile = [&](size_t tile, u32x4 (&v)[kVecPerThread]) {
        const size_t base = tile * kTileVec + threadIdx.x;
#pragma unroll
        for (int j = 0; j < kVecPerThread; ++j) {
            const size_t i = base + (size_t)j * kThreads;
            v[j] = (i < nvec && tile < tiles) ? x4[i] : u32x4{0u, 0u, 0u, 0u};
        }
    };
    auto tile_max = [&](size_t first_tile, size_t stride) -> uint32_t {
        uint32_t m = 0;
        for (size_t tile = first_tile; tile < tiles; tile += stride) {
            u32x4 v[kVecPerThread];
            load_tile(tile, v);
            m = fold(m, v);
        }
        return m;
    };
    // The first kKeep tiles of a workgroup stay in registers from the first phase to the second: a tensor of a few
    // tiles per workgroup is read once.
    constexpr int kKeep = 2;
    u32x4 kept[kKeep][kVecPerThread];
    uint32_t own = 0;
#pragma unroll
    for (int k = 0; k < kKeep; ++k) load_tile(blockIdx.x + (size_t)k * gridDim.x, kept[k]);
    copy.store(lut);  // published by the barriers of the first phase
#pragma unroll
    for (int k = 0; k < kKeep; ++k) own = fold(own, kept[k]);
    own = max(own, tile_max(blockIdx.x + (size_t)kKeep * gridDim.x, gridDim.x));
    if (blockIdx.x == 0) {
        const size_t i = nvec * 4 + threadIdx.x;
        if (i < n) own = max(own, __float_as_uint(x[i]) & 0x7fffffffu);
    }
    const uint32_t m = block_max(own, red);
    if (threadIdx.x == 0) {
        const uint32_t left = gridDim.x - group * kTicketGroup;
        const uint32_t members = left < (uint32_t)kTicketGroup ? left : (uint32_t)kTicketGroup;
        uint32_t *first = tickets + (1 + group) * kTicketStride, *second = tickets;
        uint32_t key = m;
        // a grid of one workgroup still publishes: the wait below is the same for every grid
        if ((gridDim.x == 1 || ticket_arrive(first, m, members, fenced, &key)) &&
            (groups == 1 || ticket_arrive(second, key, groups, fenced, &key))) {
            // everyone has arrived, hence read the call number: publish, then advance it
            const unsigned long long word = ((unsigned long long)call << 32) | key;
            for (uint32_t g = 0; g < groups; ++g)
                __hip_atomic_store(reinterpret_cast<unsigned long long *>(tickets + (1 + g) * kTicketStride + kResultWord), word,
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&tickets[kCallWord], call, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            precision_out[0] = __uint_as_float(key);
        }
        const unsigned long long *mine = reinterpret_cast<const unsigned long long *>(first + kResultWord);
        unsigned long long seen = __hip_atomic_load(mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        uint32_t spins = 0;
        while ((uint32_t)(seen >> 32) != call && spins < spin_limit) {
            __builtin_amdgcn_s_sleep(2);
            ++spins;
            seen = __hip_atomic_load(mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        s_complete = (uint32_t)(seen >> 32) == call ? 1u : 0u;
        s_key = (uint32_t)seen;
    }
    __syncthreads();
    uint32_t key = s_key;
    if (!s_complete) {  // uniform over the workgroup
        __syncthreads();  // `red` and s_key are reused
        uint32_t all = tile_max(0, 1);
        const size_t i = nvec * 4 + threadIdx.x;
        if (i < n) all = max(all, __float_as_uint(x[i]) & 0x7fffffffu);
        key = block_max(all, red);
        if (threadIdx.x == 0) s_key = key;
        __syncthreads();
        key = s_key;
    }
    const float precision = __uint_as_float(key);
    const double scale = quotient_scale(precision);
    const uint32_t first_of_one = xlut_first(1.0f);
    auto encode = [&](uint32_t bits) -> uint32_t { return encode_by_quotient(bits, scale, lut, first_of_one); };
    uint32_t *c4 = reinterpret_cast<uint32_t *>(codes);
    auto encode_tile = [&](size_t tile, const u32x4 (&v)[kVecPerThread]) {
        const size_t base = tile * kTileVec + threadIdx.x;
#pragma unroll
        for (int j = 0; j < kVecPerThread; ++j) {
            const size_t i = base + (size_t)j * kThreads;
            const uint32_t packed = encode(v[j].x) | (encode(v[j].y) << 8) | (encode(v[j].z) << 16) | (encode(v[j].w) << 24);
            if (i < nvec && tile < tiles) __builtin_nontemporal_store(packed, &c4[i]);
        }
    };
#pragma unroll
    for (int k = 0; k < kKeep; ++k) encode_tile(blockIdx.x + (size_t)k * gridDim.x, kept[k]);
    for (size_t tile = blockIdx.x + (size_t)kKeep * gridDim.x; tile < tiles; tile += gridDim.x) {
        u32x4 v[kVecPerThread];
        load_tile(tile, v);
        encode_tile(tile, v);
    }
    if (blockIdx.x == 0) {
        const size_t i = nvec * 4 + threadIdx.x;
        if (i < n) codes[i] = (uint8_t)encode(__float_as_uint(x[i]));
    }
}

__global__ void set_scalar_kernel(float *out, float v) {
    if (threadIdx.x == 0 && blockIdx.x == 0) out[0] = v;
}

__global__ __launch_bounds__(kThreads) void fill_kernel(float *__restrict__ dst, float v, size_t n) {
    for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (size_t)gridDim.x * kThreads)
        dst[i] = v;
}

// zeros / ones / fill of a 16-byte aligned array (source/basicOps.cu:162-165,394-407): a pure write stream, so the tiles
// are handed out in order like those of every stream that writes: a workgroup per tile of 128 KiB, or, beyond the
// cache, a persistent grid that draws them (7.2 TB/s on arithmetic-free kernels, against 6.6 TB/s grid-stride).
template <int kLanes, int kVecs, bool kDrawn>
__global__ __launch_bounds__(kLanes) void fill_tiles_kernel(float *__restrict__ dst, float v, size_t n, uint32_t *queue) {
    __shared__ uint32_t slots[2];
    const size_t nvec = n / 4;
    const uint32_t bits = __float_as_uint(v);
    const u32x4 o = {bits, bits, bits, bits};
    walk_tiles<kLanes * kVecs, kDrawn>(nvec, queue, slots, [&](size_t first) {
        const size_t left = nvec - first;
        const rsrc_t r = tile_rsrc(dst + first * 4, (uint32_t)(left < (size_t)(kLanes * kVecs) ? left : (size_t)(kLanes * kVecs)) * 16u);
#pragma unroll
        for (int j = 0; j < kVecs; ++j) __builtin_amdgcn_raw_buffer_store_b128(o, r, (j * kLanes + threadIdx.x) * 16u, 0, kAuxSc0Sc1Nt);
    });
    if (blockIdx.x == 0) {
        const size_t i = nvec * 4 + threadIdx.x;
        if (i < n) dst[i] = v;
    }
}

// Test kernel: over `count` consecutive bit patterns of x from `first`, how often the quotient the table encoder forms
// ((float)((double)x * (1.0 / (double)p)), cn_encode_table.h) differs from the division x / p.  Two NaNs count as equal, and
// so do two results below the normal range (every such quotient has the code 254).
__global__ __launch_bounds__(256) void quotient_check_kernel(uint32_t first, unsigned long long count, float p,
                                                             unsigned long long *__restrict__ mismatches) {
    const double scale = quotient_scale(p);
    unsigned long long bad = 0;
    for (unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < count;
         i += (unsigned long long)gridDim.x * blockDim.x) {
        const float x = __uint_as_float(first + (uint32_t)i);
        const uint32_t by_division = __float_as_uint(x / p);
        const uint32_t by_product = __float_as_uint((float)((double)x * scale));
        const uint32_t ma = by_division & 0x7fffffffu, mb = by_product & 0x7fffffffu;
        const bool both_nan = ma > 0x7f800000u && mb > 0x7f800000u;
        const bool both_tiny = ma < 0x00800000u && mb < 0x00800000u;
        if (by_division != by_product && !both_nan && !both_tiny) ++bad;
    }
    if (bad) atomicAdd(mismatches, bad);
}

static inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

static int g_workgroups_per_cu = 0;  // tuning hook: nonzero overrides every kernel's own figure (and keeps the tile kernels)

// Which encoder a compression takes.  Three give the same bits:
//  - the literal procedure, element by element (compress_literal_kernel): nothing to prepare, about 70 instructions and
//    nine LDS reads per element; tensors of at most kLiteralUpto elements, which are a handful of elements per lane;
//  - the table on the quotient (cn_encode_table.h): a 40 KB copy per workgroup, three more instructions per element;
//  - the table for the call's precision (build_table): about 9 000 cycles per workgroup before the first element, the
//    fewest instructions per element; tensors from kOwnTableFrom elements on, where those instructions show (819.2 M
//    elements: 622 us against 638 us) and the build does not.
// Measured, replayed from a graph, literal / quotient / own table: 2^18 elements 3.0 / 3.1 / 5.7 us; 2^20: 4.1 / 3.4 /
// 5.9; 5.12 M: 10.7 / 6.2-7.0 / 9.1-9.7; 2^23: - / 8.2 / 12.4; 26.2 M: - / 21.7-23.0 / 22.5-24.4; 2^27: - / 117 / 117.
constexpr size_t kLiteralUpto = (size_t)1 << 18;
constexpr size_t kOwnTableFrom = (size_t)1 << 27;
// Whole float4 groups from this many elements on take compress_stream_kernel (2^24 elements: 15.1 us on the tile
// kernel, 17.0 us streamed; 26.2 M: 24.5 against 23.0), and tensors with their own table draw their tiles.
constexpr size_t kStreamFrom = (size_t)20 << 20;
// With the update the streamed form exists for tensors beyond the 256 MB Infinity Cache only (2^26 elements of fp32).
constexpr size_t kBeyondCacheFrom = (size_t)1 << 26;
enum Encoder { kBySize = 0, kLiteral = 1, kQuotientTable = 2, kOwnTable = 3 };
static int g_encoder = kBySize;  // test hook (cn_host_codec_encoder): one encoder for every size

static int stream_grid(const Context *ctx, size_t n, int per_cu) {
    size_t tiles = (n / 4 + kTileVec - 1) / kTileVec;
    if (g_workgroups_per_cu > 0) per_cu = g_workgroups_per_cu;
    size_t cap = (size_t)ctx->num_cu * per_cu;
    if (cap > (size_t)kReduceSlots) cap = kReduceSlots;
    size_t g = tiles < cap ? tiles : cap;
    return (int)(g < 1 ? 1 : g);
}

template <typename Kernel>
static cn_status with_table_space(Kernel kernel, int bytes) {
    CN_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
    return CN_OK;
}

static cn_status compress_impl(const char *who, const float *x, float precision, const float *precision_dev, size_t n,
                               uint8_t *codes, float alpha, float *y, void *stream) {
    if (n == 0) return CN_OK;
    if (!x || !codes) { set_error("%s: NULL pointer", who); return CN_ERR_NULL; }
    Context *ctx;
    cn_status s = current_context(&ctx);
    if (s != CN_OK) return s;
    hipStream_t st = (hipStream_t)stream;
    const int lds_all = (int)sizeof(EncodeShared) + 256 * (int)sizeof(float);  // with the update's decode table
    const int lds = (int)sizeof(EncodeShared) + (y ? 256 * (int)sizeof(float) : 0);
    static OncePerDevice configured;
    if (configured.first(ctx->device)) {
        cn_status c = CN_OK;
        if (c == CN_OK) c = with_table_space(&compress_kernel<true, false, false>, lds_all);
        if (c == CN_OK) c = with_table_space(&compress_kernel<false, false, false>, lds_all);
        if (c == CN_OK) c = with_table_space(&compress_kernel<true, true, false>, lds_all);
        if (c == CN_OK) c = with_table_space(&compress_kernel<false, true, false>, lds_all);
        if (c == CN_OK) c = with_table_space(&compress_kernel<true, false, true>, lds_all);
        if (c == CN_OK) c = with_table_space(&compress_kernel<false, false, true>, lds_all);
        if (c == CN_OK) c = with_table_space(&compress_kernel<true, true, true>, lds_all);
        if (c == CN_OK) c = with_table_space(&compress_kernel<false, true, true>, lds_all);
        if (c == CN_OK) c = with_table_space(&compress_stream_kernel<1024, 12, false, false>, lds_all);
        if (c == CN_OK) c = with_table_space(&compress_stream_kernel<1024, 12, false, true>, lds_all);
        if (c == CN_OK) c = with_table_space(&compress_stream_kernel<512, 10, false, false>, lds_all);
        if (c == CN_OK) c = with_table_space(&compress_stream_kernel<512, 10, false, true>, lds_all);
        if (c == CN_OK) c = with_table_space(&compress_stream_kernel<1024, 4, true, false>, lds_all);
        if (c == CN_OK) c = with_table_space(&compress_stream_kernel<1024, 4, true, true>, lds_all);
        if (c != CN_OK) return c;
    }
    const bool vec = aligned(x, 16) && aligned(codes, 4) && (!y || aligned(y, 16));
    const bool tuned = g_workgroups_per_cu != 0;  // the tuning hook keeps the tile kernel and its grid
    int encoder = g_encoder;
    if (encoder == kBySize) encoder = (n <= kLiteralUpto && !tuned) ? kLiteral : n < kOwnTableFrom ? kQuotientTable : kOwnTable;
    if (encoder == kLiteral) {
        const size_t items = vec ? (n + 3) / 4 : n;
        size_t wgs = (items + kThreads - 1) / kThreads;
        const size_t cap = (size_t)ctx->num_cu * 8;
        if (wgs > cap) wgs = cap;
        auto small = y ? (vec ? compress_literal_kernel<true, true> : compress_literal_kernel<false, true>)
                       : (vec ? compress_literal_kernel<true, false> : compress_literal_kernel<false, false>);
        hipLaunchKernelGGL(small, dim3((unsigned)wgs), dim3(kThreads), 0, st, x, precision, precision_dev, n, codes,
                           ctx->table, alpha, y);
        CN_HIP(hipGetLastError());
        return CN_OK;
    }
    const bool q = encoder == kQuotientTable;
    const bool beyond_cache = n >= kBeyondCacheFrom && n < ((size_t)1 << 40);
    if (vec && n >= kStreamFrom && !tuned && (!y || beyond_cache)) {
        // One workgroup of 1024 lanes per compute unit and tiles of 192 KiB drawn from the counter for tensors that
        // stream from HBM (819.2 M elements: 620 us; 1024 x 8: 626 us, 1024 x 16: 640 us, 512 x 16: 686 us, and 639 us for
        // 256 x 12 on a grid-stride walk; tiles of 48 KiB would draw tickets faster than one counter hands them out);
        // two workgroups of 512 x 10 per compute unit on a grid-stride walk below that (2^27 elements: 117 us either
        // way; 2^26: 59 us against 66 us drawn; 2^28: 239 us against 217 us drawn).
        // With the update (x and y read, codes and y written): tiles of 1024 x 4 vectors of each array, drawn, 1.60 ms
        // on 819.2 M elements (512 x 4: 1.59 to 1.61, 512 x 6: 1.63, 512 x 8: 1.65, 512 x 12: 1.69; the tile kernel on
        // a resident grid-stride grid: 1.96 ms).
        const bool drawn = n >= kOwnTableFrom && n < ((size_t)1 << 40);
        auto launch = [&](auto kernel, int wgs, int lanes, uint32_t *queue) {
            hipLaunchKernelGGL(kernel, dim3(wgs), dim3(lanes), lds, st, x, precision, precision_dev, n, codes, ctx->xsteps,
                               ctx->xstep_count, ctx->table, queue, alpha, y, ctx->quotient_table);
        };
        uint32_t *const counter = (y || drawn) ? ctx->tile_counter_for(st) : nullptr;  // NULL: a grid-stride walk instead
        if (y) {
            if (q) launch(&compress_stream_kernel<1024, 4, true, true>, ctx->num_cu, 1024, counter);
            else   launch(&compress_stream_kernel<1024, 4, true, false>, ctx->num_cu, 1024, counter);
        } else if (drawn && counter) {
            if (q) launch(&compress_stream_kernel<1024, 12, false, true>, ctx->num_cu, 1024, counter);
            else   launch(&compress_stream_kernel<1024, 12, false, false>, ctx->num_cu, 1024, counter);
        } else {
            if (q) launch(&compress_stream_kernel<512, 10, false, true>, ctx->num_cu * 2, 512, nullptr);
            else   launch(&compress_stream_kernel<512, 10, false, false>, ctx->num_cu * 2, 512, nullptr);
        }
        CN_HIP(hipGetLastError());
        return CN_OK;
    }
    // Three workgroups per compute unit, which is what the table's LDS lets a compute unit hold: the whole grid is
    // resident at once, and the kernel keeps its own next tile in flight to stay busy at that occupancy.
    const int grid = stream_grid(ctx, n, 3);
    auto kernel = q ? (y ? (vec ? compress_kernel<true, true, true> : compress_kernel<false, true, true>)
                         : (vec ? compress_kernel<true, false, true> : compress_kernel<false, false, true>))
                    : (y ? (vec ? compress_kernel<true, true, false> : compress_kernel<false, true, false>)
                         : (vec ? compress_kernel<true, false, false> : compress_kernel<false, false, false>));
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), lds, st, x, precision, precision_dev, n, codes, ctx->xsteps,
                       ctx->xstep_count, ctx->table, alpha, y, ctx->quotient_table);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

static cn_status decompress_impl(const uint8_t *codes, float precision, const float *precision_dev,
                                 size_t n, float *out, void *stream, const float *given_lut = nullptr) {
    if (n == 0) return CN_OK;
    if (!codes || !out) { set_error("%s: NULL pointer", given_lut ? "decode_8bit_lut" : "decompress_8bit"); return CN_ERR_NULL; }
    Context *ctx;
    cn_status s = current_context(&ctx);
    if (s != CN_OK) return s;
    hipStream_t st = (hipStream_t)stream;
    // Tile shape measured on 819.2 M elements (a workgroup per tile each): 512 lanes x 2 words 590 us, 256 x 2 620 us,
    // 256 x 4 700 us, 512 x 4 760 us, 768 x 2 706 us, 1024 x 2 700 us, one word per lane 830 to 900 us; the
    // persistent one-workgroup-per-compute-unit form it replaces 672 us.  512 x 2 is also the fastest at 5.12 M
    // (4.5 us against 5.1 us) and at 26 M elements (16.5 us against 18.5 us).
    constexpr int kT = 512, kU = 2;
    const size_t wgs = (n / 4 + (size_t)kT * kU - 1) / ((size_t)kT * kU);
    if (aligned(codes, 4) && aligned(out, 16) && wgs <= 0x7fffffffu)
        hipLaunchKernelGGL((decompress_tile_kernel<kT, kU>), dim3((unsigned)(wgs < 1 ? 1 : wgs)), dim3(kT), 0, st, codes,
                           precision, precision_dev, n, out, ctx->table, given_lut);
    else
        hipLaunchKernelGGL(decompress_kernel, dim3(stream_grid(ctx, n, 8)), dim3(kThreads), 0, st, codes, precision,
                           precision_dev, n, out, ctx->table, given_lut);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

}  // namespace cn

using namespace cn;

extern "C" {

// Tuning hook: largest element count that compression encodes with the literal procedure instead of a table (0 = never, SIZE_MAX = the library's own threshold).
long long cn_host_quotient_mismatches(float precision, uint32_t first_pattern, unsigned long long patterns) {
    Context *ctx;
    if (current_context(&ctx) != CN_OK) return -1;
    unsigned long long *count = reinterpret_cast<unsigned long long *>(ctx->sum_scratch);  // 8 KB of scratch, idle here
    if (hipMemset(count, 0, sizeof(*count)) != hipSuccess) return -1;
    hipLaunchKernelGGL(quotient_check_kernel, dim3(ctx->num_cu * 8), dim3(256), 0, (hipStream_t)0, first_pattern, patterns, precision, count);
    unsigned long long host = 0;
    if (hipMemcpy(&host, count, sizeof(host), hipMemcpyDeviceToHost) != hipSuccess) return -1;
    return (long long)host;
}
void cn_host_codec_encoder(int which) { g_encoder = (which >= kBySize && which <= kOwnTable) ? which : kBySize; }

// Tuning hook: workgroups per compute unit for the codec and abs-max kernels, 0 = each kernel's own choice.
void cn_host_codec_workgroups_per_cu(int per_cu) { g_workgroups_per_cu = per_cu > 0 ? per_cu : 0; }

cn_status cn_compress_8bit(const float *x, float precision, size_t n, uint8_t *codes, void *stream) {
    return compress_impl("compress_8bit", x, precision, nullptr, n, codes, 0.0f, nullptr, stream);
}

cn_status cn_compress_8bit_dp(const float *x, const float *precision_device, size_t n, uint8_t *codes,
                              void *stream) {
    if (n != 0 && !precision_device) { set_error("compress_8bit_dp: NULL precision"); return CN_ERR_NULL; }
    return compress_impl("compress_8bit_dp", x, 0.0f, precision_device, n, codes, 0.0f, nullptr, stream);
}

cn_status cn_compress_8bit_axpy(const float *x, float precision, size_t n, uint8_t *codes, float alpha, float *y,
                                void *stream) {
    if (n != 0 && !y) { set_error("compress_8bit_axpy: NULL pointer"); return CN_ERR_NULL; }
    return compress_impl("compress_8bit_axpy", x, precision, nullptr, n, codes, alpha, y, stream);
}

cn_status cn_compress_8bit_axpy_dp(const float *x, const float *precision_device, size_t n, uint8_t *codes, float alpha,
                                   float *y, void *stream) {
    if (n != 0 && (!precision_device || !y)) { set_error("compress_8bit_axpy_dp: NULL pointer"); return CN_ERR_NULL; }
    return compress_impl("compress_8bit_axpy_dp", x, 0.0f, precision_device, n, codes, alpha, y, stream);
}

cn_status cn_decompress_8bit(const uint8_t *codes, float precision, size_t n, float *out, void *stream) {
    return decompress_impl(codes, precision, nullptr, n, out, stream);
}

cn_status cn_decompress_8bit_dp(const uint8_t *codes, const float *precision_device, size_t n, float *out,
                                void *stream) {
    if (n != 0 && !precision_device) { set_error("decompress_8bit_dp: NULL precision"); return CN_ERR_NULL; }
    return decompress_impl(codes, 0.0f, precision_device, n, out, stream);
}

cn_status cn_decode_8bit_lut(const uint8_t *codes, const float *lut256_device, size_t n, float *out, void *stream) {
    if (n != 0 && !lut256_device) { set_error("decode_8bit_lut: NULL table"); return CN_ERR_NULL; }
    return decompress_impl(codes, 0.0f, nullptr, n, out, stream, lut256_device);
}

cn_status cn_absmax_f32(const float *x, size_t n, float *out, void *stream) {
    if (!out) { set_error("absmax_f32: NULL output"); return CN_ERR_NULL; }
    Context *ctx;
    cn_status s = current_context(&ctx);
    if (s != CN_OK) return s;
    hipStream_t st = (hipStream_t)stream;
    if (n == 0) {
        // the reference's reduction starts from -1 and returns it for an empty range
        hipLaunchKernelGGL(set_scalar_kernel, dim3(1), dim3(64), 0, st, out, -1.0f);
        CN_HIP(hipGetLastError());
        return CN_OK;
    }
    if (!x) { set_error("absmax_f32: NULL input"); return CN_ERR_NULL; }
    int grid = stream_grid(ctx, n, 2);
    if (aligned(x, 16))
        hipLaunchKernelGGL((absmax_kernel<true, true>), dim3(grid), dim3(kThreads), 0, st, x, n, out, ctx->tickets, g_reduction_fences);
    else
        hipLaunchKernelGGL((absmax_kernel<false, true>), dim3(grid), dim3(kThreads), 0, st, x, n, out, ctx->tickets, g_reduction_fences);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

constexpr uint32_t kSpinLimit = 1u << 14;
static uint32_t g_absmax_compress_spins = kSpinLimit;  // test hook: 0 makes every workgroup that has to wait give up at once
// The single launch against the two stream-ordered kernels, replayed from a graph: 4 096 elements 4.3 us against 5.2;
// 0.8 M: 7.6 against 7.7; 5.12 M: 10.8 against 12.3; 2^23: 14.6 against 16.1; 2^24: 31 against 26; 26 M: 45 against 40.
// Up to 2^23 elements a workgroup's tiles stay in registers between the phases and the tensor is read once; beyond
// that the second read and the wait across the grid (a chain of round trips to the device's coherence point) cost
// more than a second launch, which is nearly free back to back.  (With a table that had to be built for the maximum
// found, the single launch was slower at every size; its table now does not depend on the precision and is
// in LDS before the wait.)
constexpr size_t kSingleLaunchUpto = (size_t)1 << 23;
static int g_absmax_compress_single_launch = -1;  // test hook: 0 never, 1 wherever it can run, -1 by size

cn_status cn_absmax_compress_8bit(const float *x, size_t n, uint8_t *codes, float *precision_out, void *stream) {
    if (!precision_out) { set_error("absmax_compress_8bit: NULL output for the precision"); return CN_ERR_NULL; }
    if (n != 0 && (!x || !codes)) { set_error("absmax_compress_8bit: NULL pointer"); return CN_ERR_NULL; }
    Context *ctx;
    cn_status s = current_context(&ctx);
    if (s != CN_OK) return s;
    hipStream_t st = (hipStream_t)stream;
    // Inputs that are empty, not aligned for 16-byte loads or too large (see above; when asked for, up to what the
    // caches can serve on the second read) take the two kernels, one behind the other on the stream.
    const bool single = g_absmax_compress_single_launch < 0 ? n <= kSingleLaunchUpto : g_absmax_compress_single_launch != 0;
    if (!single || n == 0 || n >= kBeyondCacheFrom || !aligned(x, 16) || !aligned(codes, 4)) {
        s = cn_absmax_f32(x, n, precision_out, stream);
        if (s != CN_OK || n == 0) return s;
        return cn_compress_8bit_dp(x, precision_out, n, codes, stream);
    }
    constexpr int kTableBytes = kXEntries * (int)sizeof(XEntry);
    static int resident_per_cu[kMaxDevices] = {};
    int &per_cu = resident_per_cu[ctx->device];
    if (per_cu == 0) {
        CN_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&absmax_compress_kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, kTableBytes));
        int blocks = 0;
        CN_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, reinterpret_cast<const void *>(&absmax_compress_kernel),
                                                            kThreads, kTableBytes));
        if (blocks < 1) { set_error("absmax_compress_8bit: the kernel does not fit a compute unit"); return CN_ERR_HIP; }
        per_cu = blocks > 2 ? 2 : blocks;
    }
    const size_t tiles = (n / 4 + kTileVec - 1) / kTileVec;
    size_t grid = (size_t)ctx->num_cu * per_cu;  // resident as a whole: the wait inside the kernel relies on it
    if (grid > tiles) grid = tiles;
    if (grid < 1) grid = 1;
    hipLaunchKernelGGL(absmax_compress_kernel, dim3((unsigned)grid), dim3(kThreads), kTableBytes, st, x, n, codes,
                       precision_out, ctx->tickets, g_absmax_compress_spins, ctx->quotient_table, g_reduction_fences);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

void cn_host_absmax_compress_single_launch(int mode) { g_absmax_compress_single_launch = mode < 0 ? -1 : mode != 0; }

void cn_host_absmax_compress_spin_limit(int spins) { g_absmax_compress_spins = spins < 0 ? kSpinLimit : (uint32_t)spins; }

cn_status cn_max_f32(const float *x, size_t n, float *out, void *stream) {
    if (!out) { set_error("max_f32: NULL output"); return CN_ERR_NULL; }
    Context *ctx;
    cn_status s = current_context(&ctx);
    if (s != CN_OK) return s;
    hipStream_t st = (hipStream_t)stream;
    if (n == 0) {
        hipLaunchKernelGGL(set_scalar_kernel, dim3(1), dim3(64), 0, st, out, -1.0f);
        CN_HIP(hipGetLastError());
        return CN_OK;
    }
    if (!x) { set_error("max_f32: NULL input"); return CN_ERR_NULL; }
    int grid = stream_grid(ctx, n, 2);
    if (aligned(x, 16))
        hipLaunchKernelGGL((absmax_kernel<true, false>), dim3(grid), dim3(kThreads), 0, st, x, n, out, ctx->tickets, g_reduction_fences);
    else
        hipLaunchKernelGGL((absmax_kernel<false, false>), dim3(grid), dim3(kThreads), 0, st, x, n, out, ctx->tickets, g_reduction_fences);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

cn_status cn_fill_f32(float *dst, float value, size_t n, void *stream) {
    if (n == 0) return CN_OK;
    if (!dst) { set_error("fill_f32: NULL pointer"); return CN_ERR_NULL; }
    Context *ctx;
    cn_status s = current_context(&ctx);
    if (s != CN_OK) return s;
    constexpr int kFillLanes = 1024, kFillVecs = 8;
    const size_t tiles = (n / 4 + (size_t)kFillLanes * kFillVecs - 1) / ((size_t)kFillLanes * kFillVecs);
    uint32_t *const counter = (aligned(dst, 16) && n >= kDrawnFrom && n < kDrawnBelow) ? ctx->tile_counter_for((hipStream_t)stream) : nullptr;
    if (counter) {
        hipLaunchKernelGGL((fill_tiles_kernel<kFillLanes, kFillVecs, true>), dim3(ctx->num_cu), dim3(kFillLanes), 0, (hipStream_t)stream,
                           dst, value, n, counter);
    } else if (aligned(dst, 16) && n >= ((size_t)1 << 20) && tiles <= 0x7fffffffu) {
        hipLaunchKernelGGL((fill_tiles_kernel<kFillLanes, kFillVecs, false>), dim3((unsigned)tiles), dim3(kFillLanes), 0,
                           (hipStream_t)stream, dst, value, n, (uint32_t *)nullptr);
    } else {
        size_t blocks = (n + kThreads - 1) / kThreads;
        size_t cap = (size_t)ctx->num_cu * 16;
        int grid = (int)(blocks < cap ? blocks : cap);
        hipLaunchKernelGGL(fill_kernel, dim3(grid), dim3(kThreads), 0, (hipStream_t)stream, dst, value, n);
    }
    CN_HIP(hipGetLastError());
    return CN_OK;
}

}  // extern "C"
