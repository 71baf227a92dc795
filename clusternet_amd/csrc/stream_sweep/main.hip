// stream_sweep <out.csv> [kind | -1] [repetitions]: times every variant (sweep.h) under every mapping, occupancy
// and store-wait setting on the 100000 x 8192 gradient's 819.2 M elements, together with the HIP runtime's own
// copy and fill as yardsticks from outside.  summarize.py turns the CSV into the table kept under profiles/.
#include <stdio.h>
#include <stdlib.h>

#include <algorithm>

#include "sweep.h"

#define CK(x)                                                                       \
    do {                                                                            \
        hipError_t e_ = (x);                                                        \
        if (e_ != hipSuccess) {                                                     \
            fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                 \
            exit(2);                                                                \
        }                                                                           \
    } while (0)

__global__ void fill_random(uint32_t *p, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        uint32_t x = (uint32_t)i * 2654435761u;
        x ^= x >> 15;
        x *= 0x85ebca6bu;
        x ^= x >> 13;
        p[i] = (x & 0x807fffffu) | 0x3c800000u;  // magnitude about 0.02, random mantissa and sign
    }
}

int main(int argc, char **argv) {
    const char *path = argc > 1 ? argv[1] : "stream_sweep.csv";
    const int only_kind = argc > 2 ? atoi(argv[2]) : -1;
    const int reps = argc > 3 ? atoi(argv[3]) : 3;
    std::vector<Variant> v;
    register_kind_0(v); register_kind_1(v); register_kind_2(v); register_kind_3(v);
    register_kind_4(v); register_kind_5(v); register_kind_6(v);
    hipDeviceProp_t prop;
    CK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    const size_t n = 819200000;
    void *f32a, *f32b, *bytes;
    uint32_t *sink;
    CK(hipMalloc(&f32a, n * 4));
    CK(hipMalloc(&f32b, n * 4));
    CK(hipMalloc(&bytes, n));
    CK(hipMalloc((void **)&sink, (size_t)cus * 64 * 1024 * 4));
    fill_random<<<cus * 8, 256>>>((uint32_t *)f32a, n);
    fill_random<<<cus * 8, 256>>>((uint32_t *)bytes, n / 4);
    CK(hipDeviceSynchronize());
    FILE *f = fopen(path, "w");
    if (!f) { fprintf(stderr, "cannot write %s\n", path); return 2; }
    fprintf(f, "kind,load_policy,store_policy,U,T,chunk_tiles,xcd_remap,wait_for_stores,waves_per_cu,grid,min_ms,med_ms,GBps_min,GBps_med\n");
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    hipStream_t st = 0;
    auto time_it = [&](auto &&fn) {
        std::vector<float> ms;
        fn();
        for (int r = 0; r < reps; ++r) {
            CK(hipEventRecord(e0, st));
            fn();
            CK(hipEventRecord(e1, st));
            CK(hipEventSynchronize(e1));
            float t;
            CK(hipEventElapsedTime(&t, e0, e1));
            ms.push_back(t);
        }
        std::sort(ms.begin(), ms.end());
        return std::make_pair(ms[0], ms[ms.size() / 2]);
    };
    if (only_kind < 0) {
        auto a = time_it([&] { CK(hipMemcpyAsync(f32b, f32a, n * 4, hipMemcpyDeviceToDevice, st)); });
        fprintf(f, "hipMemcpyDtoD,,,,,,,,,,%.4f,%.4f,%.1f,%.1f\n", a.first, a.second, 8.0 * n / a.first / 1e6, 8.0 * n / a.second / 1e6);
        auto b = time_it([&] { CK(hipMemsetAsync(f32b, 0x3c, n * 4, st)); });
        fprintf(f, "hipMemsetD8,,,,,,,,,,%.4f,%.4f,%.1f,%.1f\n", b.first, b.second, 4.0 * n / b.first / 1e6, 4.0 * n / b.second / 1e6);
        auto c = time_it([&] { CK(hipMemsetD32Async((hipDeviceptr_t)f32b, 0x3c000000, n, st)); });
        fprintf(f, "hipMemsetD32,,,,,,,,,,%.4f,%.4f,%.1f,%.1f\n", c.first, c.second, 4.0 * n / c.first / 1e6, 4.0 * n / c.second / 1e6);
        fflush(f);
    }
    size_t done = 0;
    for (const Variant &k : v) {
        if (only_kind >= 0 && k.kind != only_kind) continue;
        const uint32_t tile_floats = (uint32_t)k.T * k.U * 4;
        const uint32_t tiles = (uint32_t)(n / tile_floats);  // a few tiles' worth at the end stays untouched when U is 12
        const bool from_bytes = k.kind == R1W4 || k.kind == R1W4W, to_bytes = k.kind == R4W1 || k.kind == R4W1W;
        const void *in = from_bytes ? bytes : f32a;
        void *out = to_bytes ? bytes : f32b;
        const uint32_t ib = from_bytes ? (uint32_t)n : (uint32_t)(n * 4), ob = to_bytes ? (uint32_t)n : (uint32_t)(n * 4);
        const double moved = (double)tiles * tile_floats * ((k.kind == R4 || k.kind == W4) ? 4.0 : (k.kind == R4W4 ? 8.0 : 5.0));
        // One tile per workgroup, as many workgroups as tiles, placed by the dispatcher as compute units free up
        // (waves_per_cu 0 in the file): the shape of an ordinary element-wise launch.
        for (int wait = 0; wait < (k.kind == R4 ? 1 : 2); ++wait) {
            auto t = time_it([&] { k.go(tiles, st, in, out, ib, ob, tiles, 1, 0, wait, sink); });
            fprintf(f, "%d,%d,%d,%d,%d,%u,%d,%d,%d,%u,%.4f,%.4f,%.1f,%.1f\n", k.kind, k.load_policy, k.store_policy, k.U, k.T, 1u, 0,
                    wait, 0, tiles, t.first, t.second, moved / t.first / 1e6, moved / t.second / 1e6);
        }
        if (k.U < 4) continue;  // the short tiles are there for the launch above only
        for (int waves : {4, 8, 16, 32, 64}) {
            const int per_cu = waves / (k.T / 64);
            if (per_cu < 1) continue;
            const unsigned grid = (unsigned)(cus * per_cu);
            const uint32_t two_mib = std::max(1u, (2u << 20) / (tile_floats * 4));
            const uint32_t full = (tiles + grid - 1) / grid;
            struct Map { uint32_t chunk; int remap; } maps[] = {{1, 0}, {two_mib, 0}, {two_mib, 1}, {full, 0}, {full, 1}, {1, 2}};
            for (const Map &m : maps)
                for (int wait = 0; wait < (k.kind == R4 ? 1 : 2); ++wait) {
                    auto t = time_it([&] { k.go(grid, st, in, out, ib, ob, tiles, m.chunk, m.remap, wait, sink); });
                    fprintf(f, "%d,%d,%d,%d,%d,%u,%d,%d,%d,%u,%.4f,%.4f,%.1f,%.1f\n", k.kind, k.load_policy, k.store_policy, k.U, k.T,
                            m.chunk, m.remap, wait, waves, grid, t.first, t.second, moved / t.first / 1e6, moved / t.second / 1e6);
                }
        }
        CK(hipGetLastError());
        if (++done % 20 == 0) {
            fflush(f);
            printf("variants done: %zu of %zu\n", done, v.size());
            fflush(stdout);
        }
    }
    fclose(f);
    printf("sweep complete: %zu variants\n", done);
    return 0;
}
