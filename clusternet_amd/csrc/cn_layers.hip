// Small element-wise / layout kernels the callers of the GEMM + codec path use around it: layout
// transpose, scalar affine map, sum, bias broadcast, maxout with arg-max, its gradient scatter,
// row softmax, difference, and a plain gradient step.  All row-major, all HBM-bound streaming
// kernels; none of them is on the measured hot path.
#include <float.h>

#include "cn_internal.h"
#include "cn_tile_queue.h"

namespace cn {

constexpr int kT = 256;
typedef float f32x4_t __attribute__((ext_vector_type(4)));

static inline int grid_for(const Context *ctx, int64_t work_items, int per_cu = 8) {
    int64_t blocks = (work_items + kT - 1) / kT;
    int64_t cap = (int64_t)ctx->num_cu * per_cu;
    if (blocks > cap) blocks = cap;
    return (int)(blocks < 1 ? 1 : blocks);
}

// out[c][r] = in[r][c] on square tiles of kEdge = 64 or 128 through LDS, a workgroup of kEdge^2 / 16 lanes per tile.  Whole
// tiles of 16-byte aligned matrices move as 16-byte vectors on both sides (256 or 512 contiguous bytes per tile row); the
// tiles are numbered down the columns of `in`, so that workgroups started one after the other write neighbouring
// pieces of the same kEdge rows of `out`: the stream that writes is the one that needs its window narrow.  On 64 x 64
// tiles 4.3 TB/s (32 x 32 tiles of single floats) became 4.9 to 5.3 TB/s on a 100000 x 8192 matrix and 4.2 became 5.5 to
// 5.7 on 20000 x 40000; 128 x 128 tiles (twice the contiguous bytes per row on either side, 66 KB of LDS) give 5.5 and 5.7
// there and 6.1 instead of 5.5 on 8192 x 100096 (128 x 64 tiles: 5.3 / 5.5 / 6.1; 64 x 128: 5.0 / 5.5 / 5.6; 32 x 256 and
// 256 x 32 in between), so matrices with a thousand and more of them take those.
template <int kEdge, bool kVector>
__global__ __launch_bounds__(kEdge * kEdge / 16) void transpose_tile_kernel(const float *__restrict__ in, int64_t rows, int64_t cols,
                                                                            float *__restrict__ out, int64_t tiles_r) {
    extern __shared__ float tile[];  // kEdge rows of kEdge + 1 floats
    constexpr int kPitch = kEdge + 1, kLanes = kEdge * kEdge / 16;
    const int64_t tc = blockIdx.x / tiles_r, tr = blockIdx.x % tiles_r;
    const int64_t r0 = tr * kEdge, c0 = tc * kEdge;
    if (kVector && r0 + kEdge <= rows && c0 + kEdge <= cols) {
        constexpr int kAcross = kEdge / 4, kDown = kLanes / kAcross;  // vectors across, rows down, four passes
        const int tx = threadIdx.x % kAcross, ty = threadIdx.x / kAcross;
#pragma unroll
        for (int j = 0; j < kEdge / kDown; ++j) {
            const int r = ty + kDown * j;
            const f32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t *>(in + (r0 + r) * cols + c0 + 4 * tx));
            tile[r * kPitch + 4 * tx + 0] = v.x;
            tile[r * kPitch + 4 * tx + 1] = v.y;
            tile[r * kPitch + 4 * tx + 2] = v.z;
            tile[r * kPitch + 4 * tx + 3] = v.w;
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < kEdge / kDown; ++j) {
            const int c = ty + kDown * j;
            const f32x4_t o = {tile[(4 * tx + 0) * kPitch + c], tile[(4 * tx + 1) * kPitch + c], tile[(4 * tx + 2) * kPitch + c],
                               tile[(4 * tx + 3) * kPitch + c]};
            __builtin_nontemporal_store(o, reinterpret_cast<f32x4_t *>(out + (c0 + c) * rows + r0 + 4 * tx));
        }
    } else {
        constexpr int kDown = kLanes / kEdge;  // kEdge single floats across, kDown rows down
        const int tx = threadIdx.x % kEdge, ty = threadIdx.x / kEdge;
#pragma unroll 4
        for (int j = 0; j < kEdge; j += kDown) {
            const int64_t r = r0 + ty + j, c = c0 + tx;
            if (r < rows && c < cols) tile[(ty + j) * kPitch + tx] = in[r * cols + c];
        }
        __syncthreads();
#pragma unroll 4
        for (int j = 0; j < kEdge; j += kDown) {
            const int64_t c = c0 + ty + j, r = r0 + tx;
            if (r < rows && c < cols) out[c * rows + r] = tile[tx * kPitch + ty + j];
        }
    }
}

// The same on 128 x 128 tiles by a persistent grid (a workgroup of 1024 lanes per compute unit) that draws its tiles in
// that order from a counter: the loads of a workgroup's next tile are in flight while it stores the current one.
__global__ __launch_bounds__(1024) void transpose_drawn_kernel(const float *__restrict__ in, int64_t rows, int64_t cols,
                                                               float *__restrict__ out, int64_t tiles_r, uint32_t tiles,
                                                               uint32_t *__restrict__ counter) {
    extern __shared__ float tile[];  // 128 rows of 129 floats
    __shared__ uint32_t queue_slots[2];
    constexpr int kEdge = 128, kPitch = kEdge + 1, kAcross = kEdge / 4, kDown = 1024 / kAcross;
    const int tx = threadIdx.x % kAcross, ty = threadIdx.x / kAcross;
    const int sx = threadIdx.x % kEdge, sy = threadIdx.x / kEdge;  // the element-wise form of ragged tiles: 128 across, 8 down
    f32x4_t v[kEdge / kDown];
    auto whole = [&](uint32_t t) {
        const int64_t r0 = (int64_t)(t % tiles_r) * kEdge, c0 = (int64_t)(t / tiles_r) * kEdge;
        return r0 + kEdge <= rows && c0 + kEdge <= cols;
    };
    auto request = [&](uint32_t t) {
        const int64_t r0 = (int64_t)(t % tiles_r) * kEdge, c0 = (int64_t)(t / tiles_r) * kEdge;
#pragma unroll
        for (int j = 0; j < kEdge / kDown; ++j)
            v[j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t *>(in + (r0 + ty + kDown * j) * cols + c0 + 4 * tx));
    };
    TileQueue q = tile_queue(counter, tiles, queue_slots);
    q.draw_ahead();
    uint32_t cur = q.next();
    if (cur < tiles) q.draw_ahead();  // every workgroup draws exactly one ticket past the last tile
    if (cur < tiles && whole(cur)) request(cur);
    while (cur < tiles) {
        const int64_t r0 = (int64_t)(cur % tiles_r) * kEdge, c0 = (int64_t)(cur / tiles_r) * kEdge;
        const bool is_whole = whole(cur);
        if (is_whole) {
#pragma unroll
            for (int j = 0; j < kEdge / kDown; ++j) {
                float *row = tile + (ty + kDown * j) * kPitch + 4 * tx;
                row[0] = v[j].x; row[1] = v[j].y; row[2] = v[j].z; row[3] = v[j].w;
            }
        } else {
            for (int j = 0; j < kEdge; j += 8) {
                const int64_t r = r0 + sy + j, c = c0 + sx;
                if (r < rows && c < cols) tile[(sy + j) * kPitch + sx] = in[r * cols + c];
            }
        }
        const uint32_t nxt = q.next();  // a barrier: the tile is in LDS
        if (nxt < tiles) q.draw_ahead();
        if (nxt < tiles && whole(nxt)) request(nxt);
        if (is_whole) {
#pragma unroll
            for (int j = 0; j < kEdge / kDown; ++j) {
                const int c = ty + kDown * j;
                const f32x4_t o = {tile[(4 * tx + 0) * kPitch + c], tile[(4 * tx + 1) * kPitch + c], tile[(4 * tx + 2) * kPitch + c],
                                   tile[(4 * tx + 3) * kPitch + c]};
                __builtin_nontemporal_store(o, reinterpret_cast<f32x4_t *>(out + (c0 + c) * rows + r0 + 4 * tx));
            }
        } else {
            for (int j = 0; j < kEdge; j += 8) {
                const int64_t c = c0 + sy + j, r = r0 + sx;
                if (r < rows && c < cols) out[c * rows + r] = tile[sx * kPitch + sy + j];
            }
        }
        __syncthreads();  // everyone has read the tile before the next one is written
        cur = nxt;
    }
}

// out[c][r] = in[r][c]; 32 x 32 tiles through LDS (33-float pitch), both sides coalesced.
__global__ __launch_bounds__(kT) void transpose_kernel(const float *__restrict__ in, int64_t rows, int64_t cols,
                                                       float *__restrict__ out) {
    __shared__ float tile[32][33];
    const int64_t tiles_c = (cols + 31) / 32, tiles_r = (rows + 31) / 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    for (int64_t t = blockIdx.x; t < tiles_c * tiles_r; t += gridDim.x) {
        const int64_t r0 = (t / tiles_c) * 32, c0 = (t % tiles_c) * 32;
#pragma unroll
        for (int j = 0; j < 32; j += 8) {
            int64_t r = r0 + ty + j, c = c0 + tx;
            if (r < rows && c < cols) tile[ty + j][tx] = in[r * cols + c];
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 32; j += 8) {
            int64_t c = c0 + ty + j, r = r0 + tx;
            if (r < rows && c < cols) out[c * rows + r] = tile[tx][ty + j];
        }
        __syncthreads();
    }
}

// Flat element-wise passes: out[i] = f(a[i], b[i]).  With 16-byte aligned arrays every lane moves 16-byte vectors
// (non-temporal: nothing is reused) and the tiles are handed out in order, so that the tiles in flight lie next to one
// another in memory: a workgroup per tile and as many workgroups as tiles, or, beyond the cache, a persistent grid that
// draws its tiles from a counter (the weight update on 819.2 M elements: 6.7 TB/s drawn, 6.1 TB/s with a workgroup per
// tile, 5.5 TB/s on a persistent grid-stride grid).  Otherwise, and for the last n % 4 elements, element by element.
// Each f is the single fp32 expression of its reference routine.
struct AffineOp { float mul, add; __device__ float operator()(float x, float) const { return x * mul + add; } };
struct AbsOp { __device__ float operator()(float x, float) const { return fabsf(x); } };
struct SubOp { __device__ float operator()(float a, float b) const { return a - b; } };
struct SgdOp { float rate; __device__ float operator()(float w, float g) const { return w - rate * g; } };

template <class Op, bool kTwo, bool kVector, int kLanes, int kVecs, bool kDrawn>
__global__ __launch_bounds__(kLanes) void flat_kernel(const float *a, const float *b, int64_t n, float *out, Op f,
                                                       uint32_t *queue) {
    if (kVector) {
        __shared__ uint32_t slots[2];
        const size_t nvec = (size_t)n / 4;
        const f32x4_t *a4 = reinterpret_cast<const f32x4_t *>(a), *b4 = reinterpret_cast<const f32x4_t *>(b);
        f32x4_t *o4 = reinterpret_cast<f32x4_t *>(out);
        walk_tiles<kLanes * kVecs, kDrawn>(nvec, queue, slots, [&](size_t first) {
            const size_t base = first + threadIdx.x;
            f32x4_t va[kVecs], vb[kVecs];
#pragma unroll
            for (int j = 0; j < kVecs; ++j) {
                const size_t i = base + (size_t)j * kLanes;
                va[j] = i < nvec ? __builtin_nontemporal_load(&a4[i]) : f32x4_t{0.f, 0.f, 0.f, 0.f};
                if (kTwo) vb[j] = i < nvec ? __builtin_nontemporal_load(&b4[i]) : f32x4_t{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int j = 0; j < kVecs; ++j) {
                const size_t i = base + (size_t)j * kLanes;
                f32x4_t o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = f(va[j][e], kTwo ? vb[j][e] : 0.0f);
                if (i < nvec) __builtin_nontemporal_store(o, &o4[i]);
            }
        });
        if (blockIdx.x == 0) {
            const int64_t i = (int64_t)nvec * 4 + threadIdx.x;
            if (i < n) out[i] = f(a[i], kTwo ? b[i] : 0.0f);
        }
    } else {
        for (int64_t i = (int64_t)blockIdx.x * kLanes + threadIdx.x; i < n; i += (int64_t)gridDim.x * kLanes)
            out[i] = f(a[i], kTwo ? b[i] : 0.0f);
    }
}

template <class Op, bool kTwo>
static cn_status launch_flat(Context *ctx, hipStream_t st, const float *a, const float *b, int64_t n, float *out, Op f) {
    auto ok16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
    const bool vec = ok16(a) && ok16(out) && (!kTwo || ok16(b));
    constexpr int kFT = 512;
    uint32_t *const counter = (vec && (size_t)n >= kDrawnFrom && (size_t)n < kDrawnBelow) ? ctx->tile_counter_for(st) : nullptr;
    if (counter) {
        // beyond the cache: one workgroup per compute unit, tiles of 512 lanes x 8 vectors drawn from the counter (the
        // weight update on 819.2 M elements: 1.46 ms; 1024 x 4: 1.48, 256 x 16: 1.50, 512 x 4: 1.49, 1024 x 8: 1.58)
        hipLaunchKernelGGL((flat_kernel<Op, kTwo, true, kFT, 8, true>), dim3(ctx->num_cu), dim3(kFT), 0, st, a, b, n, out, f,
                           counter);
    } else if (vec) {
        // a workgroup per tile of 512 lanes x 2 vectors, as many workgroups as tiles
        int64_t grid = (n / 4 + kFT * 2 - 1) / (kFT * 2);
        grid = grid < 1 ? 1 : (grid > 0x7fffffff ? 0x7fffffff : grid);
        hipLaunchKernelGGL((flat_kernel<Op, kTwo, true, kFT, 2, false>), dim3((unsigned)grid), dim3(kFT), 0, st, a, b, n, out, f,
                           (uint32_t *)nullptr);
    } else {
        int64_t blocks = (n + kT - 1) / kT, cap = (int64_t)ctx->num_cu * 8;
        const int64_t grid = blocks < 1 ? 1 : (blocks < cap ? blocks : cap);
        hipLaunchKernelGGL((flat_kernel<Op, kTwo, false, kT, 1, false>), dim3((unsigned)grid), dim3(kT), 0, st, a, b, n, out, f,
                           (uint32_t *)nullptr);
    }
    CN_HIP(hipGetLastError());
    return CN_OK;
}

// out[r][c] = A[r][c] + v[c]
__global__ __launch_bounds__(kT) void add_row_vector_kernel(const float *__restrict__ A, const float *__restrict__ v,
                                                            int64_t rows, int64_t cols, float *__restrict__ out) {
    const int64_t n = rows * cols;
    for (int64_t i = (int64_t)blockIdx.x * kT + threadIdx.x; i < n; i += (int64_t)gridDim.x * kT)
        out[i] = A[i] + v[i % cols];
}

// Maxout over `pool` consecutive columns; arg-max is the absolute column index as a float, the
// first maximum wins (strict comparison, as the reference's reduction).
__global__ __launch_bounds__(kT) void maxout_kernel(const float *__restrict__ A, int64_t rows, int64_t cols, int pool,
                                                    float *__restrict__ out, float *__restrict__ argmax) {
    const int64_t oc = cols / pool, n = rows * oc;
    for (int64_t i = (int64_t)blockIdx.x * kT + threadIdx.x; i < n; i += (int64_t)gridDim.x * kT) {
        const int64_t r = i / oc, o = i % oc;
        const float *src = A + r * cols + o * pool;
        float best = src[0];
        int arg = 0;
        for (int p = 1; p < pool; ++p) {
            float v = src[p];
            if (best < v) { best = v; arg = p; }
        }
        out[i] = best;
        argmax[i] = (float)(o * pool + arg);
    }
}

// maxout_kernel on A + v (v added to every row) in one pass: the sums are formed, compared and dropped.
__global__ __launch_bounds__(kT) void bias_maxout_kernel(const float *__restrict__ A, int64_t lda,
                                                         const float *__restrict__ v, int64_t rows, int64_t cols, int pool,
                                                         float *__restrict__ out, float *__restrict__ argmax) {
    const int64_t oc = cols / pool, n = rows * oc;
    for (int64_t i = (int64_t)blockIdx.x * kT + threadIdx.x; i < n; i += (int64_t)gridDim.x * kT) {
        const int64_t r = i / oc, o = i % oc;
        const float *src = A + r * lda + o * pool;
        const float *bias = v + o * pool;
        float best = src[0] + bias[0];
        int arg = 0;
        for (int p = 1; p < pool; ++p) {
            const float z = src[p] + bias[p];
            if (best < z) { best = z; arg = p; }
        }
        out[i] = best;
        argmax[i] = (float)(o * pool + arg);
    }
}

// out (rows x pooled*pool): the pooled error lands on the winner's column, zero elsewhere.
__global__ __launch_bounds__(kT) void expand_maxout_grad_kernel(const float *__restrict__ err,
                                                                const float *__restrict__ argmax, int64_t rows,
                                                                int64_t pooled, int pool, float *__restrict__ out) {
    const int64_t cols = pooled * pool, n = rows * cols;
    for (int64_t i = (int64_t)blockIdx.x * kT + threadIdx.x; i < n; i += (int64_t)gridDim.x * kT) {
        const int64_t r = i / cols, c = i % cols;
        const int64_t o = c / pool;
        out[i] = ((int64_t)argmax[r * pooled + o] == c) ? err[r * pooled + o] : 0.0f;
    }
}

// One wavefront per row: max, sum of exp, normalise.
__global__ __launch_bounds__(kT) void softmax_kernel(const float *__restrict__ A, int64_t rows, int64_t cols,
                                                     float *__restrict__ out) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = ((int64_t)blockIdx.x * kT + threadIdx.x) >> 6;
    const int64_t nwaves = ((int64_t)gridDim.x * kT) >> 6;
    for (int64_t r = wave; r < rows; r += nwaves) {
        const float *src = A + r * cols;
        float m = -FLT_MAX;
        for (int64_t c = lane; c < cols; c += 64) m = fmaxf(m, src[c]);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
        float s = 0.0f;
        for (int64_t c = lane; c < cols; c += 64) s += expf(src[c] - m);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
        for (int64_t c = lane; c < cols; c += 64) out[r * cols + c] = expf(src[c] - m) / s;
    }
}

// Deterministic two-stage sum in fp64: fixed grid, per-workgroup partials, the last workgroup to arrive folds
// them in a fixed order.  A partial is published with a device-scope exchange and the arrival count is made
// to depend on what the exchange returned, so the partial has been stored before the workgroup is counted:
// ordering by data dependence, which costs far less than a fence per workgroup.
__global__ __launch_bounds__(kT) void sum_kernel(const float *__restrict__ x, int64_t n, float *__restrict__ out,
                                                 double *__restrict__ partial, uint32_t *__restrict__ counter, int fenced) {
    __shared__ double sm[kT];
    __shared__ uint32_t s_last;
    double s = 0.0;
    const int64_t tid = (int64_t)blockIdx.x * kT + threadIdx.x, stride = (int64_t)gridDim.x * kT;
    if ((reinterpret_cast<uintptr_t>(x) & 15) == 0) {
        // 16-byte loads, four running sums per lane, two vectors in flight; the order is fixed by the grid
        typedef float f32x4 __attribute__((ext_vector_type(4)));
        const f32x4 *x4 = reinterpret_cast<const f32x4 *>(x);
        const int64_t nvec = n / 4;
        double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
        int64_t i = tid;
        for (; i + stride < nvec; i += 2 * stride) {
            const f32x4 a = __builtin_nontemporal_load(&x4[i]), b = __builtin_nontemporal_load(&x4[i + stride]);
            s0 += (double)a.x; s1 += (double)a.y; s2 += (double)a.z; s3 += (double)a.w;
            s0 += (double)b.x; s1 += (double)b.y; s2 += (double)b.z; s3 += (double)b.w;
        }
        if (i < nvec) {
            const f32x4 a = __builtin_nontemporal_load(&x4[i]);
            s0 += (double)a.x; s1 += (double)a.y; s2 += (double)a.z; s3 += (double)a.w;
        }
        s = (s0 + s1) + (s2 + s3);
        if (tid < n - 4 * nvec) s += (double)x[4 * nvec + tid];
    } else {
        for (int64_t i = tid; i < n; i += stride) s += (double)x[i];
    }
    sm[threadIdx.x] = s;
    __syncthreads();
    for (int w = kT / 2; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) sm[threadIdx.x] += sm[threadIdx.x + w];
        __syncthreads();
    }
    unsigned long long *slots = reinterpret_cast<unsigned long long *>(partial);
    if (threadIdx.x == 0) {
        const unsigned long long before = atomicExch(&slots[blockIdx.x], (unsigned long long)__double_as_longlong(sm[0]));
        uint32_t one = 1u;
        asm volatile("" : "+v"(one) : "v"(before));  // `one` is not available before `before` is
        // writer side: ordered by that dependence (see absmax_kernel), or by a release fence when `fenced`
        if (fenced) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        const uint32_t ticket = atomicAdd(counter, one);
        s_last = (ticket == gridDim.x - 1) ? 1u : 0u;
        // reader side: the last to arrive acquires before any of its lanes reads the partial sums
        if (s_last) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    }
    __syncthreads();
    if (s_last) {
        // every thread fetches its share of the partials (independent loads), then the same tree as above
        double t = 0.0;
        for (uint32_t b = threadIdx.x; b < gridDim.x; b += kT)
            t += __longlong_as_double((long long)__hip_atomic_load(&slots[b], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
        sm[threadIdx.x] = t;
        __syncthreads();
        for (int w = kT / 2; w > 0; w >>= 1) {
            if ((int)threadIdx.x < w) sm[threadIdx.x] += sm[threadIdx.x + w];
            __syncthreads();
        }
        if (threadIdx.x == 0) {
            out[0] = (float)sm[0];
            __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

}  // namespace cn

using namespace cn;

#define CN_ENTER(name)                                   \
    Context *ctx;                                        \
    {                                                    \
        cn_status s_ = current_context(&ctx);            \
        if (s_ != CN_OK) return s_;                      \
    }                                                    \
    hipStream_t st = (hipStream_t)stream;                \
    (void)st;

#define CN_REQUIRE(cond, code, msg)                      \
    do {                                                 \
        if (!(cond)) { set_error("%s", msg); return code; } \
    } while (0)

extern "C" {

cn_status cn_transpose_f32(const float *in, int64_t rows, int64_t cols, float *out, void *stream) {
    CN_REQUIRE(rows >= 0 && cols >= 0, CN_ERR_SHAPE, "transpose_f32: negative dimension");
    if (rows == 0 || cols == 0) return CN_OK;
    CN_REQUIRE(in && out, CN_ERR_NULL, "transpose_f32: NULL pointer");
    CN_REQUIRE(in != out, CN_ERR_ARG, "transpose_f32: in-place transpose is not supported");
    CN_ENTER();
    auto ok16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
    const bool vec = ok16(in) && ok16(out) && rows % 4 == 0 && cols % 4 == 0;
    auto tiled = [&](auto kernel, int edge) -> cn_status {
        const int lds = edge * (edge + 1) * (int)sizeof(float);
        static OncePerDevice configured[2][2];
        if (configured[edge == 128][vec].first(ctx->device))
            CN_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        const int64_t tiles_r = (rows + edge - 1) / edge, tiles = tiles_r * ((cols + edge - 1) / edge);
        hipLaunchKernelGGL(kernel, dim3((unsigned)tiles), dim3(edge * edge / 16), lds, st, in, rows, cols, out, tiles_r);
        CN_HIP(hipGetLastError());
        return CN_OK;
    };
    const int64_t tiles128 = ((rows + 127) / 128) * ((cols + 127) / 128);
    uint32_t *const counter = (vec && (size_t)rows * (size_t)cols >= kDrawnFrom && tiles128 <= 0x7fffffffLL) ? ctx->tile_counter_for(st) : nullptr;
    if (counter) {
        // beyond the cache: a persistent workgroup per compute unit draws the tiles in the same order and has its next
        // tile's loads in flight while it stores (100000 x 8192: 5.9 TB/s against 5.5 for a workgroup per tile; 20000 x
        // 40000: 5.8 against 5.5; 8192 x 100096: 6.15 either way; 4096 x 4096: 31 us against 24, hence the bound)
        const int lds = 128 * 129 * (int)sizeof(float);
        static OncePerDevice drawn_configured;
        if (drawn_configured.first(ctx->device))
            CN_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&transpose_drawn_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        hipLaunchKernelGGL(transpose_drawn_kernel, dim3(ctx->num_cu), dim3(1024), lds, st, in, rows, cols, out, (rows + 127) / 128,
                           (uint32_t)tiles128, counter);
        CN_HIP(hipGetLastError());
        return CN_OK;
    }
    if (tiles128 >= 1024 && tiles128 <= 0x7fffffffLL)
        return vec ? tiled(&transpose_tile_kernel<128, true>, 128) : tiled(&transpose_tile_kernel<128, false>, 128);
    if (rows * cols >= (1 << 16) && tiles128 <= 0x7fffffffLL / 4)
        return vec ? tiled(&transpose_tile_kernel<64, true>, 64) : tiled(&transpose_tile_kernel<64, false>, 64);
    int64_t tiles = ((rows + 31) / 32) * ((cols + 31) / 32);
    int64_t cap = (int64_t)ctx->num_cu * 8;
    hipLaunchKernelGGL(transpose_kernel, dim3((unsigned)(tiles < cap ? tiles : cap)), dim3(kT), 0, st, in, rows, cols, out);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

cn_status cn_affine_f32(const float *x, float mul, float add, size_t n, float *out, void *stream) {
    if (n == 0) return CN_OK;
    CN_REQUIRE(x && out, CN_ERR_NULL, "affine_f32: NULL pointer");
    CN_ENTER();
    return launch_flat<AffineOp, false>(ctx, st, x, nullptr, (int64_t)n, out, AffineOp{mul, add});
}

cn_status cn_abs_f32(const float *x, size_t n, float *out, void *stream) {
    if (n == 0) return CN_OK;
    CN_REQUIRE(x && out, CN_ERR_NULL, "abs_f32: NULL pointer");
    CN_ENTER();
    return launch_flat<AbsOp, false>(ctx, st, x, nullptr, (int64_t)n, out, AbsOp{});
}

cn_status cn_sub_f32(const float *a, const float *b, size_t n, float *out, void *stream) {
    if (n == 0) return CN_OK;
    CN_REQUIRE(a && b && out, CN_ERR_NULL, "sub_f32: NULL pointer");
    CN_ENTER();
    return launch_flat<SubOp, true>(ctx, st, a, b, (int64_t)n, out, SubOp{});
}

cn_status cn_sgd_update_f32(float *w, const float *grad, float rate, size_t n, void *stream) {
    if (n == 0) return CN_OK;
    CN_REQUIRE(w && grad, CN_ERR_NULL, "sgd_update_f32: NULL pointer");
    CN_ENTER();
    return launch_flat<SgdOp, true>(ctx, st, w, grad, (int64_t)n, w, SgdOp{rate});
}

cn_status cn_add_row_vector_f32(const float *A, const float *v, int64_t rows, int64_t cols, float *out, void *stream) {
    CN_REQUIRE(rows >= 0 && cols >= 0, CN_ERR_SHAPE, "add_row_vector_f32: negative dimension");
    if (rows == 0 || cols == 0) return CN_OK;
    CN_REQUIRE(A && v && out, CN_ERR_NULL, "add_row_vector_f32: NULL pointer");
    CN_ENTER();
    hipLaunchKernelGGL(add_row_vector_kernel, dim3(grid_for(ctx, rows * cols)), dim3(kT), 0, st, A, v, rows, cols, out);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

cn_status cn_maxout_f32(const float *A, int64_t rows, int64_t cols, int pool, float *out, float *argmax, void *stream) {
    CN_REQUIRE(rows >= 0 && cols >= 0 && pool >= 1, CN_ERR_SHAPE, "maxout_f32: bad dimension");
    CN_REQUIRE(cols % pool == 0, CN_ERR_SHAPE, "maxout_f32: columns are not a multiple of the pool size");
    if (rows == 0 || cols == 0) return CN_OK;
    CN_REQUIRE(A && out && argmax, CN_ERR_NULL, "maxout_f32: NULL pointer");
    CN_ENTER();
    hipLaunchKernelGGL(maxout_kernel, dim3(grid_for(ctx, rows * (cols / pool))), dim3(kT), 0, st, A, rows, cols, pool, out, argmax);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

cn_status cn_bias_maxout_f32(const float *A, int64_t lda, const float *v, int64_t rows, int64_t cols, int pool, float *out,
                             float *argmax, void *stream) {
    CN_REQUIRE(rows >= 0 && cols >= 0 && pool >= 1 && lda >= cols, CN_ERR_SHAPE, "bias_maxout_f32: bad dimension");
    CN_REQUIRE(cols % pool == 0, CN_ERR_SHAPE, "bias_maxout_f32: columns are not a multiple of the pool size");
    if (rows == 0 || cols == 0) return CN_OK;
    CN_REQUIRE(A && v && out && argmax, CN_ERR_NULL, "bias_maxout_f32: NULL pointer");
    CN_ENTER();
    hipLaunchKernelGGL(bias_maxout_kernel, dim3(grid_for(ctx, rows * (cols / pool))), dim3(kT), 0, st, A, lda, v, rows, cols, pool,
                       out, argmax);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

cn_status cn_expand_to_maxout_grad_f32(const float *err, const float *argmax, int64_t rows, int64_t pooled_cols,
                                       int pool, float *out, void *stream) {
    CN_REQUIRE(rows >= 0 && pooled_cols >= 0 && pool >= 1, CN_ERR_SHAPE, "expand_to_maxout_grad_f32: bad dimension");
    if (rows == 0 || pooled_cols == 0) return CN_OK;
    CN_REQUIRE(err && argmax && out, CN_ERR_NULL, "expand_to_maxout_grad_f32: NULL pointer");
    CN_ENTER();
    hipLaunchKernelGGL(expand_maxout_grad_kernel, dim3(grid_for(ctx, rows * pooled_cols * pool)), dim3(kT), 0, st,
                       err, argmax, rows, pooled_cols, pool, out);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

cn_status cn_softmax_f32(const float *A, int64_t rows, int64_t cols, float *out, void *stream) {
    CN_REQUIRE(rows >= 0 && cols >= 0, CN_ERR_SHAPE, "softmax_f32: negative dimension");
    if (rows == 0 || cols == 0) return CN_OK;
    CN_REQUIRE(A && out, CN_ERR_NULL, "softmax_f32: NULL pointer");
    CN_ENTER();
    hipLaunchKernelGGL(softmax_kernel, dim3(grid_for(ctx, rows * 64)), dim3(kT), 0, st, A, rows, cols, out);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

cn_status cn_sum_f32(const float *x, size_t n, float *out_device, void *stream) {
    CN_REQUIRE(out_device, CN_ERR_NULL, "sum_f32: NULL output");
    CN_REQUIRE(n == 0 || x, CN_ERR_NULL, "sum_f32: NULL input");
    CN_ENTER();
    // every workgroup ends with two returning atomics on shared words, some 12 ns each and one after the other:
    // two workgroups per CU (four for an input of 256 MB and more, where the tail no longer counts), and for a
    // small input one per 16384 elements
    int grid = grid_for(ctx, (int64_t)(n ? (n + 63) / 64 : 1), n >= ((size_t)64 << 20) ? 4 : 2);
    if (grid > 1024) grid = 1024;
    // arrival counter: the slot after the abs-max kernel's counter
    hipLaunchKernelGGL(sum_kernel, dim3(grid), dim3(kT), 0, st, x, (int64_t)n, out_device, ctx->sum_scratch,
                       ctx->reduce_scratch + kReduceSlots + 1, g_reduction_fences);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

// Stopwatch on a stream (hipEvent pair), the counterpart of the reference's tick/tock helpers
// (source/util.cu:218-252).
struct cn_timer { hipEvent_t start, stop; };

cn_status cn_timer_start(void **handle, void *stream) {
    CN_REQUIRE(handle, CN_ERR_NULL, "timer_start: NULL handle");
    cn_timer *t = new cn_timer;
    CN_HIP(hipEventCreate(&t->start));
    CN_HIP(hipEventCreate(&t->stop));
    CN_HIP(hipEventRecord(t->start, (hipStream_t)stream));
    *handle = t;
    return CN_OK;
}

cn_status cn_timer_stop(void *handle, void *stream, float *milliseconds) {
    CN_REQUIRE(handle && milliseconds, CN_ERR_NULL, "timer_stop: NULL pointer");
    cn_timer *t = static_cast<cn_timer *>(handle);
    CN_HIP(hipEventRecord(t->stop, (hipStream_t)stream));
    CN_HIP(hipEventSynchronize(t->stop));
    CN_HIP(hipEventElapsedTime(milliseconds, t->start, t->stop));
    CN_HIP(hipEventDestroy(t->start));
    CN_HIP(hipEventDestroy(t->stop));
    delete t;
    return CN_OK;
}

}  // extern "C"
