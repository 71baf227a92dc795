// Fused passes over a weight gradient and its weights for gfx950: the steps that follow the 8-bit
// exchange of a gradient in the reference, each as one HBM-bound streaming kernel instead of two or
// three.
//   decompress_axpy   y += alpha * decode(codes)            1 + 4 B read, 4 B written per element
//                     (decompression_8bit followed by add / sub / a scaled update: 17 B)
//   rmsprop_update    RMSprop with weight update             12 B read (9 with coded gradient), 8 B written
//                     (decompression_8bit followed by the update: 25 B)
// Every arithmetic step is a separate fp32 operation in the order the unfused kernels use, so the
// results equal theirs bit for bit.
#include "cn_internal.h"
#include "cn_tile_queue.h"

namespace cn {

namespace {

// Arrays of whole 16-byte vectors are walked tile by tile with the tiles handed out in order (cn_tile_queue.h), which a
// stream that also writes needs on this part: a workgroup per tile of 512 lanes x 2 vectors and as many workgroups as
// tiles, or, beyond the cache, one persistent workgroup per compute unit that draws tiles of 512 x kDrawnVecs vectors
// from a counter and waits for a tile's stores before it takes the next.  The weight update on 819.2 M elements: 1.46 ms drawn, 1.62 ms with a workgroup per tile, 1.79 ms
// on a persistent grid-stride grid.
constexpr int kThreads = 512;
constexpr int kTileVecsSmall = 2;

typedef float f32x4 __attribute__((ext_vector_type(4)));

// 256-entry decode table of kDecompression_8bit (source/clusterKernels.cu:1135-1160), each entry
// multiplied by `alpha` afterwards (alpha = 1 leaves the plain table).
__device__ __forceinline__ void build_lut(float *lut, const float *table, float precision, float alpha) {
    const int t = threadIdx.x;
    if (t < 126) {
        float v = table[t] * precision;
        lut[t] = alpha * v;
        lut[t + 128] = alpha * (-v);
    } else if (t == 126) {
        lut[126] = alpha * precision;
        lut[127] = alpha * precision;
        lut[254] = alpha * precision;
        lut[255] = alpha * (-precision);
    }
    __syncthreads();
}

// y[i] = y[i] + alpha * decode(codes[i])
template <bool kVector, int kVecs, bool kDrawn>
__global__ __launch_bounds__(kThreads) void decompress_axpy_kernel(
    const uint8_t *__restrict__ codes, float precision_value, const float *__restrict__ precision_ptr,
    float alpha, size_t n, float *__restrict__ y, const float *__restrict__ table, uint32_t *queue) {
    __shared__ float lut[256];
    __shared__ uint32_t slots[2];
    build_lut(lut, table, precision_ptr ? *precision_ptr : precision_value, alpha);
    if (kVector) {
        const size_t nvec = n / 4;
        const uint32_t *c4 = reinterpret_cast<const uint32_t *>(codes);
        f32x4 *y4 = reinterpret_cast<f32x4 *>(y);
        walk_tiles<kThreads * kVecs, kDrawn>(nvec, queue, slots, [&](size_t first) {
            const size_t base = first + threadIdx.x;
            uint32_t w[kVecs];
            f32x4 v[kVecs];
#pragma unroll
            for (int j = 0; j < kVecs; ++j) {
                const size_t i = base + (size_t)j * kThreads;
                w[j] = (i < nvec) ? __builtin_nontemporal_load(&c4[i]) : 0u;
                v[j] = (i < nvec) ? __builtin_nontemporal_load(&y4[i]) : f32x4{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int j = 0; j < kVecs; ++j) {
                const size_t i = base + (size_t)j * kThreads;
                f32x4 o;
                o.x = v[j].x + lut[w[j] & 0xffu];
                o.y = v[j].y + lut[(w[j] >> 8) & 0xffu];
                o.z = v[j].z + lut[(w[j] >> 16) & 0xffu];
                o.w = v[j].w + lut[w[j] >> 24];
                if (i < nvec) __builtin_nontemporal_store(o, &y4[i]);
            }
        });
        if (blockIdx.x == 0) {
            const size_t i = nvec * 4 + threadIdx.x;
            if (i < n) y[i] = y[i] + lut[codes[i]];
        }
    } else {
        for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (size_t)gridDim.x * kThreads)
            y[i] = y[i] + lut[codes[i]];
    }
}

// One element of kRMSprop_with_weight_update (source/clusterKernels.cu:1305-1325).  powf(g, 2) is
// g * g; fdividef is written as a division.
__device__ __forceinline__ void rmsprop_one(float g, float &rms, float &w, float mult, float one_minus, float rate) {
    const float r = (mult * rms) + ((g * g) * one_minus);
    const float step = rate * (g / (sqrtf(r) + 1.0e-08f));
    rms = r;
    w = w - step;
}

template <bool kCoded, bool kVector, int kVecs, bool kDrawn>
__global__ __launch_bounds__(kThreads) void rmsprop_update_kernel(
    float *__restrict__ rms, const float *__restrict__ grad, const uint8_t *__restrict__ codes,
    float precision_value, const float *__restrict__ precision_ptr, float *__restrict__ w, float mult,
    float rate, size_t n, const float *__restrict__ table, uint32_t *queue) {
    __shared__ float lut[256];
    __shared__ uint32_t slots[2];
    if (kCoded) build_lut(lut, table, precision_ptr ? *precision_ptr : precision_value, 1.0f);
    const float one_minus = 1.0f - mult;
    if (kVector) {
        const size_t nvec = n / 4;
        const uint32_t *c4 = reinterpret_cast<const uint32_t *>(codes);
        const f32x4 *g4 = reinterpret_cast<const f32x4 *>(grad);
        f32x4 *r4 = reinterpret_cast<f32x4 *>(rms);
        f32x4 *w4 = reinterpret_cast<f32x4 *>(w);
        walk_tiles<kThreads * kVecs, kDrawn>(nvec, queue, slots, [&](size_t first) {
            const size_t base = first + threadIdx.x;
            // all loads of the tile first
            f32x4 g[kVecs], r[kVecs], ww[kVecs];
            uint32_t c[kVecs];
#pragma unroll
            for (int j = 0; j < kVecs; ++j) {
                const size_t i = base + (size_t)j * kThreads;
                const bool in = i < nvec;
                if (kCoded) c[j] = in ? __builtin_nontemporal_load(&c4[i]) : 0u;
                else g[j] = in ? __builtin_nontemporal_load(&g4[i]) : f32x4{0.f, 0.f, 0.f, 0.f};
                r[j] = in ? __builtin_nontemporal_load(&r4[i]) : f32x4{0.f, 0.f, 0.f, 0.f};
                ww[j] = in ? __builtin_nontemporal_load(&w4[i]) : f32x4{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int j = 0; j < kVecs; ++j) {
                const size_t i = base + (size_t)j * kThreads;
                if (kCoded) g[j] = f32x4{lut[c[j] & 0xffu], lut[(c[j] >> 8) & 0xffu], lut[(c[j] >> 16) & 0xffu], lut[c[j] >> 24]};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float re = r[j][e], we = ww[j][e];
                    rmsprop_one(g[j][e], re, we, mult, one_minus, rate);
                    r[j][e] = re;
                    ww[j][e] = we;
                }
                if (i < nvec) {
                    __builtin_nontemporal_store(r[j], &r4[i]);
                    __builtin_nontemporal_store(ww[j], &w4[i]);
                }
            }
        });
        if (blockIdx.x == 0) {
            const size_t i = nvec * 4 + threadIdx.x;
            if (i < n) rmsprop_one(kCoded ? lut[codes[i]] : grad[i], rms[i], w[i], mult, one_minus, rate);
        }
    } else {
        for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (size_t)gridDim.x * kThreads)
            rmsprop_one(kCoded ? lut[codes[i]] : grad[i], rms[i], w[i], mult, one_minus, rate);
    }
}

inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// Vector form: a workgroup per tile.  Element-by-element form (unaligned arrays): a grid-stride loop on a resident grid.
int grid_of(const Context *ctx, size_t n, bool vec) {
    const size_t per = (size_t)kThreads * kTileVecsSmall;
    const size_t tiles = vec ? (n / 4 + per - 1) / per : (n + kThreads - 1) / kThreads;
    const size_t cap = vec ? (size_t)0x7fffffffu : (size_t)ctx->num_cu * 4;
    const size_t g = tiles < cap ? tiles : cap;
    return (int)(g < 1 ? 1 : g);
}

// Vectors per lane of a drawn tile.  Measured on 819.2 M elements, a workgroup per tile / drawn x 4 / drawn x 8:
// decode+add 1.15 / 1.31 / 1.11 ms, RMSprop 2.82 / 2.58 / 2.61 ms, RMSprop on codes 2.35 / 2.39 / 2.31 ms (tiles of
// 512 x 4 vectors draw tickets about as fast as one counter hands them out).
constexpr int kDrawnVecs = 8;

cn_status axpy_impl(const uint8_t *codes, float precision, const float *precision_dev, float alpha, size_t n,
                    float *y, void *stream) {
    if (n == 0) return CN_OK;
    if (!codes || !y) { set_error("decompress_8bit_axpy: NULL pointer"); return CN_ERR_NULL; }
    Context *ctx;
    cn_status s = current_context(&ctx);
    if (s != CN_OK) return s;
    hipStream_t st = (hipStream_t)stream;
    const bool vec = aligned(codes, 4) && aligned(y, 16);
    const int grid = grid_of(ctx, n, vec);
    uint32_t *const none = nullptr;
    uint32_t *const counter = (vec && n >= kDrawnFrom && n < kDrawnBelow) ? ctx->tile_counter_for(st) : nullptr;
    if (counter)
        hipLaunchKernelGGL((decompress_axpy_kernel<true, kDrawnVecs, true>), dim3(ctx->num_cu), dim3(kThreads), 0, st, codes,
                           precision, precision_dev, alpha, n, y, ctx->table, counter);
    else if (vec)
        hipLaunchKernelGGL((decompress_axpy_kernel<true, kTileVecsSmall, false>), dim3(grid), dim3(kThreads), 0, st, codes,
                           precision, precision_dev, alpha, n, y, ctx->table, none);
    else
        hipLaunchKernelGGL((decompress_axpy_kernel<false, 1, false>), dim3(grid), dim3(kThreads), 0, st, codes, precision,
                           precision_dev, alpha, n, y, ctx->table, none);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

cn_status rmsprop_impl(float *rms, const float *grad, const uint8_t *codes, float precision,
                       const float *precision_dev, float *w, float mult, float rate, size_t n, void *stream) {
    if (n == 0) return CN_OK;
    if (!rms || !w || (!grad && !codes)) { set_error("rmsprop_update: NULL pointer"); return CN_ERR_NULL; }
    Context *ctx;
    cn_status s = current_context(&ctx);
    if (s != CN_OK) return s;
    hipStream_t st = (hipStream_t)stream;
    const bool vec = aligned(rms, 16) && aligned(w, 16) && (codes ? aligned(codes, 4) : aligned(grad, 16));
    uint32_t *const queue = (vec && n >= kDrawnFrom && n < kDrawnBelow) ? ctx->tile_counter_for(st) : nullptr;
    const bool drawn = queue != nullptr;
    const int grid = drawn ? ctx->num_cu : grid_of(ctx, n, vec);
    auto go = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), 0, st, rms, grad, codes, precision, precision_dev, w, mult, rate, n,
                           ctx->table, queue);
    };
    if (codes) {
        if (drawn) go(rmsprop_update_kernel<true, true, kDrawnVecs, true>);
        else if (vec) go(rmsprop_update_kernel<true, true, kTileVecsSmall, false>);
        else go(rmsprop_update_kernel<true, false, 1, false>);
    } else {
        if (drawn) go(rmsprop_update_kernel<false, true, kDrawnVecs, true>);
        else if (vec) go(rmsprop_update_kernel<false, true, kTileVecsSmall, false>);
        else go(rmsprop_update_kernel<false, false, 1, false>);
    }
    CN_HIP(hipGetLastError());
    return CN_OK;
}

}  // namespace

}  // namespace cn

using namespace cn;

extern "C" {

cn_status cn_decompress_8bit_axpy(const uint8_t *codes, float precision, float alpha, size_t n, float *y,
                                  void *stream) {
    return axpy_impl(codes, precision, nullptr, alpha, n, y, stream);
}

cn_status cn_decompress_8bit_axpy_dp(const uint8_t *codes, const float *precision_device, float alpha, size_t n,
                                     float *y, void *stream) {
    if (n != 0 && !precision_device) { set_error("decompress_8bit_axpy_dp: NULL precision"); return CN_ERR_NULL; }
    return axpy_impl(codes, 0.0f, precision_device, alpha, n, y, stream);
}

cn_status cn_rmsprop_update_f32(float *rms, const float *grad, float *w, float rms_multiplier, float learning_rate,
                                size_t n, void *stream) {
    if (n != 0 && !grad) { set_error("rmsprop_update_f32: NULL gradient"); return CN_ERR_NULL; }
    return rmsprop_impl(rms, grad, nullptr, 0.0f, nullptr, w, rms_multiplier, learning_rate, n, stream);
}

cn_status cn_rmsprop_update_w8(float *rms, const uint8_t *codes, float precision, float *w, float rms_multiplier,
                               float learning_rate, size_t n, void *stream) {
    if (n != 0 && !codes) { set_error("rmsprop_update_w8: NULL codes"); return CN_ERR_NULL; }
    return rmsprop_impl(rms, nullptr, codes, precision, nullptr, w, rms_multiplier, learning_rate, n, stream);
}

cn_status cn_rmsprop_update_w8_dp(float *rms, const uint8_t *codes, const float *precision_device, float *w,
                                  float rms_multiplier, float learning_rate, size_t n, void *stream) {
    if (n != 0 && (!codes || !precision_device)) { set_error("rmsprop_update_w8_dp: NULL pointer"); return CN_ERR_NULL; }
    return rmsprop_impl(rms, nullptr, codes, 0.0f, precision_device, w, rms_multiplier, learning_rate, n, stream);
}

}  // extern "C"
