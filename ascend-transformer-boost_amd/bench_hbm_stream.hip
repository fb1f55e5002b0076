// How fast a kernel that only reads streams cache-sized windows from HBM on this device: the yardstick the attention
// kernels' bandwidth figures are read against. 256 workgroups (or more) x 4 waves read 252 MB in tiles of 36 864 bytes
// (32 rows of the 576-channel latent cache), 1 KB an instruction, from one of three windows in turn so that nothing
// stays in the 256 MB memory-side cache; the last line reads one window over and over (served from that cache).
// Build and run (the package's build step makes lib/bench_hbm_stream too):
//     hipcc -O3 -std=c++17 --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops
//         ascend-transformer-boost_amd/bench_hbm_stream.hip -o ascend-transformer-boost_amd/lib/bench_hbm_stream   (one line)
//     ascend-transformer-boost_amd/lib/bench_hbm_stream
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <cstdint>
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
#define CHECK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("error %s at %d\n", hipGetErrorString(e), __LINE__); exit(1); } } while (0)
constexpr int TILE = 36864;
// MODE 0: a workgroup reads its own contiguous region tile by tile; 1: tiles interleaved between workgroups;
// NT: non-temporal loads; DEPTH tiles in flight per thread
template <int THREADS, int MODE, bool NT, int DEPTH>
__global__ __launch_bounds__(THREADS) void Stream(const unsigned char *base, int tilesPerWg, unsigned int *sink)
{
    constexpr int PER = TILE / 16 / THREADS;           // 16-byte pieces per thread per tile (9 at 256 threads)
    static_assert(TILE % (16 * THREADS) == 0, "");
    const int wg = blockIdx.x, nwg = gridDim.x, tid = threadIdx.x;
    u32x4 acc = {0, 0, 0, 0};
    u32x4 buf[DEPTH][PER];
    auto addr = [&](int t, int i) {
        const size_t tile = MODE == 0 ? static_cast<size_t>(wg) * tilesPerWg + t : static_cast<size_t>(t) * nwg + wg;
        return reinterpret_cast<const u32x4 *>(base + tile * TILE + (static_cast<size_t>(i) * THREADS + tid) * 16);
    };
    auto load = [&](int t, u32x4 *dst) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            dst[i] = NT ? __builtin_nontemporal_load(addr(t, i)) : *addr(t, i);
        }
    };
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        if (d < tilesPerWg) load(d, buf[d]);
    }
    for (int t = 0; t < tilesPerWg; t += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            if (t + d < tilesPerWg) {
#pragma unroll
                for (int i = 0; i < PER; ++i) acc ^= buf[d][i];
                if (t + d + DEPTH < tilesPerWg) load(t + d + DEPTH, buf[d]);
            }
        }
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) sink[0] = 1;
}
template <int THREADS, int MODE, bool NT, int DEPTH> void Run(const char *name, unsigned char *buf, size_t window, int copies, unsigned int *sink, int wgs)
{
    const int tilesPerWg = static_cast<int>(window / TILE / wgs);
    hipEvent_t a, b;
    CHECK(hipEventCreate(&a)); CHECK(hipEventCreate(&b));
    for (int i = 0; i < 3; ++i) Stream<THREADS, MODE, NT, DEPTH><<<wgs, THREADS>>>(buf + (i % copies) * window, tilesPerWg, sink);
    CHECK(hipDeviceSynchronize());
    const int reps = 30;
    CHECK(hipEventRecord(a));
    for (int i = 0; i < reps; ++i) Stream<THREADS, MODE, NT, DEPTH><<<wgs, THREADS>>>(buf + (i % copies) * window, tilesPerWg, sink);
    CHECK(hipEventRecord(b));
    CHECK(hipEventSynchronize(b));
    float ms = 0; CHECK(hipEventElapsedTime(&ms, a, b));
    const double bytes = static_cast<double>(tilesPerWg) * wgs * TILE;
    printf("%-44s wgs %4d tiles/wg %3d  %.1f us  %.2f TB/s\n", name, wgs, tilesPerWg, ms / reps * 1e3, bytes / (ms / reps * 1e-3) / 1e12);
    fflush(stdout);
}
int main()
{
    const size_t window = 252ull << 20; const int copies = 3;
    unsigned char *buf; unsigned int *sink;
    CHECK(hipMalloc(&buf, window * copies)); CHECK(hipMalloc(&sink, 4));
    CHECK(hipMemset(buf, 1, window * copies)); CHECK(hipMemset(sink, 0, 4));
    Run<256, 0, false, 1>("256 thr, own region, depth 1", buf, window, copies, sink, 256);
    Run<256, 0, false, 2>("256 thr, own region, depth 2", buf, window, copies, sink, 256);
    Run<256, 0, false, 4>("256 thr, own region, depth 4", buf, window, copies, sink, 256);
    Run<256, 0, true, 2>("256 thr, own region, depth 2, nt", buf, window, copies, sink, 256);
    Run<256, 1, false, 2>("256 thr, interleaved, depth 2", buf, window, copies, sink, 256);
    Run<256, 1, true, 2>("256 thr, interleaved, depth 2, nt", buf, window, copies, sink, 256);
    Run<256, 0, false, 2>("256 thr, own region, depth 2, 512 wgs", buf, window, copies, sink, 512);
    Run<256, 0, false, 2>("256 thr, own region, depth 2, 1024 wgs", buf, window, copies, sink, 1024);
    Run<256, 0, false, 2>("256 thr, own region, depth 2, 2048 wgs", buf, window, copies, sink, 2048);
    Run<256, 0, true, 2>("256 thr, own region, depth 2, nt, 2048 wgs", buf, window, copies, sink, 2048);
    Run<256, 0, false, 2>("256 thr, own region, depth 2, 128 wgs", buf, window, copies, sink, 128);
    Run<256, 0, false, 2>("256 thr, one copy (memory-side cache)", buf, window, 1, sink, 256);
    return 0;
}
