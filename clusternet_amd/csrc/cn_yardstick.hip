// Stream kernels with the codec's access patterns and no arithmetic: what the memory system gives a
// kernel that only moves the bytes compression_8bit / decompression_8bit / abs-max have to move.
// They exist so that the codec's throughput can be read against a ceiling measured on the same
// device in the same process; nothing on the path calls them.
#include <hip/hip_runtime.h>

#include "cn_internal.h"

namespace cn {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int kT = 256;
constexpr int kLoads = 4;  // 16-byte loads in flight per lane

// kKind 0: read fp32, keep a running maximum of the bit patterns (one word written per lane at the end)
//       1: read fp32, write the top byte of each word            (4 bytes in, 1 byte out)
//       2: read bytes, write each as fp32                        (1 byte in, 4 bytes out)
//       3: copy fp32                                             (4 in, 4 out)
template <int kKind>
__global__ __launch_bounds__(kT) void stream_kernel(const void *__restrict__ in, void *__restrict__ out, size_t tiles) {
    const f32x4 *in4 = reinterpret_cast<const f32x4 *>(in);
    const uint32_t *in1 = reinterpret_cast<const uint32_t *>(in);
    uint32_t running = 0;
    for (size_t t = blockIdx.x; t < tiles; t += gridDim.x) {
        const size_t base = t * (size_t)(kT * kLoads) + threadIdx.x;
        if (kKind == 2) {
            uint32_t w[kLoads];
#pragma unroll
            for (int j = 0; j < kLoads; ++j) w[j] = __builtin_nontemporal_load(&in1[base + (size_t)j * kT]);
#pragma unroll
            for (int j = 0; j < kLoads; ++j) {
                const f32x4 o = {(float)(w[j] & 255u), (float)((w[j] >> 8) & 255u), (float)((w[j] >> 16) & 255u),
                                 (float)(w[j] >> 24)};
                __builtin_nontemporal_store(o, &reinterpret_cast<f32x4 *>(out)[base + (size_t)j * kT]);
            }
        } else {
            f32x4 v[kLoads];
#pragma unroll
            for (int j = 0; j < kLoads; ++j) v[j] = __builtin_nontemporal_load(&in4[base + (size_t)j * kT]);
#pragma unroll
            for (int j = 0; j < kLoads; ++j) {
                const uint32_t a = __float_as_uint(v[j].x), b = __float_as_uint(v[j].y), c = __float_as_uint(v[j].z),
                               d = __float_as_uint(v[j].w);
                if (kKind == 0) {
                    const uint32_t m = max(max(a, b), max(c, d));
                    running = m > running ? m : running;
                } else if (kKind == 1) {
                    const uint32_t p = (a >> 24) | ((b >> 24) << 8) | ((c >> 24) << 16) | ((d >> 24) << 24);
                    __builtin_nontemporal_store(p, &reinterpret_cast<uint32_t *>(out)[base + (size_t)j * kT]);
                } else {
                    __builtin_nontemporal_store(v[j], &reinterpret_cast<f32x4 *>(out)[base + (size_t)j * kT]);
                }
            }
        }
    }
    if (kKind == 0) reinterpret_cast<uint32_t *>(out)[(size_t)blockIdx.x * kT + threadIdx.x] = running;
}

}  // namespace
}  // namespace cn

using namespace cn;

extern "C" cn_status cn_stream_yardstick(int kind, const void *in, void *out, size_t n, int workgroups_per_cu,
                                         void *stream) {
    constexpr size_t kTileElements = (size_t)kT * kLoads * 4;
    if (kind < 0 || kind > 3 || workgroups_per_cu < 1 || workgroups_per_cu > 64) {
        set_error("stream_yardstick: kind 0..3, 1..64 workgroups per CU");
        return CN_ERR_ARG;
    }
    if (n == 0 || n % kTileElements != 0) {
        set_error("stream_yardstick: n must be a positive multiple of %zu elements", kTileElements);
        return CN_ERR_ARG;
    }
    if (!in || !out) { set_error("stream_yardstick: NULL pointer"); return CN_ERR_NULL; }
    if (reinterpret_cast<uintptr_t>(in) % 16 || reinterpret_cast<uintptr_t>(out) % 16) {
        set_error("stream_yardstick: buffers must be 16-byte aligned");
        return CN_ERR_ARG;
    }
    Context *ctx;
    cn_status s = current_context(&ctx);
    if (s != CN_OK) return s;
    hipStream_t st = (hipStream_t)stream;
    const size_t tiles = n / kTileElements;
    size_t grid = (size_t)ctx->num_cu * workgroups_per_cu;
    if (grid > tiles) grid = tiles;
    switch (kind) {
        case 0: hipLaunchKernelGGL(stream_kernel<0>, dim3((unsigned)grid), dim3(kT), 0, st, in, out, tiles); break;
        case 1: hipLaunchKernelGGL(stream_kernel<1>, dim3((unsigned)grid), dim3(kT), 0, st, in, out, tiles); break;
        case 2: hipLaunchKernelGGL(stream_kernel<2>, dim3((unsigned)grid), dim3(kT), 0, st, in, out, tiles); break;
        default: hipLaunchKernelGGL(stream_kernel<3>, dim3((unsigned)grid), dim3(kT), 0, st, in, out, tiles); break;
    }
    CN_HIP(hipGetLastError());
    return CN_OK;
}
