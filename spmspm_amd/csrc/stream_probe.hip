// Read-streaming ceiling of the GPU this runs on: a plain read of a buffer four times the size of the last-level
// cache with the load shapes the SpMM kernel could use (16 bytes per lane, 4 or 8 KB in flight per wave, 8 to 32
// waves per CU, with and without the non-temporal hint).  The best rate is what "as fast as a memcpy-like read" means
// on this machine, next to the 8 TB/s of the data sheet.  Prints a table and one JSON line.
//   hipcc -O3 --offload-arch=gfx950 stream_probe.hip -o stream_probe && ./stream_probe [MiB]
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#define CK(x)                                                                                   \
    do {                                                                                        \
        hipError_t e_ = (x);                                                                    \
        if (e_ != hipSuccess) {                                                                 \
            std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);          \
            std::exit(1);                                                                       \
        }                                                                                       \
    } while (0)

typedef unsigned uintx4 __attribute__((ext_vector_type(4)));

// Every wave owns a contiguous region and keeps kInFlight 1 KB loads outstanding.
template <bool kNonTemporal, int kInFlight>
__global__ __launch_bounds__(256) void read_stream(const char* __restrict__ src, size_t bytes_per_wave, unsigned* out)
{
    const int     lane = threadIdx.x & 63;
    const size_t  wave = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const uintx4* p    = reinterpret_cast<const uintx4*>(src + wave * bytes_per_wave) + lane;
    const size_t  n    = bytes_per_wave / 1024; // a multiple of kInFlight
    unsigned      acc  = 0;
    for (size_t i = 0; i < n; i += kInFlight) {
        uintx4 r[kInFlight];
#pragma unroll
        for (int u = 0; u < kInFlight; ++u)
            r[u] = kNonTemporal ? __builtin_nontemporal_load(p + (i + u) * 64) : p[(i + u) * 64];
#pragma unroll
        for (int u = 0; u < kInFlight; ++u)
            acc ^= r[u].x ^ r[u].w;
    }
    if (acc == 0x1234567u) // never true for the fill pattern: keeps the loads alive
        out[threadIdx.x] = acc;
}

int main(int argc, char** argv)
{
    const size_t total = (size_t)(argc > 1 ? std::atoi(argv[1]) : 1024) << 20;
    char*        src;
    unsigned*    out;
    CK(hipMalloc(&src, total));
    CK(hipMemset(src, 1, total));
    CK(hipMalloc(&out, 4096));
    hipDeviceProp_t prop;
    CK(hipGetDeviceProperties(&prop, 0));
    const int  cus = prop.multiProcessorCount;
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    double best = 0;
    char   best_name[128] = "";
    auto bench = [&](const char* name, auto kern, int waves_per_cu, int in_flight) {
        const int    nwg   = cus * waves_per_cu / 4;
        const size_t gran  = (size_t)in_flight * 1024;
        const size_t bpw   = total / ((size_t)nwg * 4) / gran * gran;
        const size_t bytes = bpw * nwg * 4;
        for (int i = 0; i < 3; ++i)
            hipLaunchKernelGGL(kern, dim3(nwg), dim3(256), 0, 0, src, bpw, out);
        CK(hipDeviceSynchronize());
        const int reps = 10;
        CK(hipEventRecord(e0));
        for (int i = 0; i < reps; ++i)
            hipLaunchKernelGGL(kern, dim3(nwg), dim3(256), 0, 0, src, bpw, out);
        CK(hipEventRecord(e1));
        CK(hipEventSynchronize(e1));
        float ms;
        CK(hipEventElapsedTime(&ms, e0, e1));
        const double gbs = (double)bytes * reps / (ms * 1e-3) / 1e9;
        std::printf("%-44s %3d waves/CU  %7.1f GB/s\n", name, waves_per_cu, gbs);
        if (gbs > best) {
            best = gbs;
            std::snprintf(best_name, sizeof best_name, "%s, %d waves/CU", name, waves_per_cu);
        }
    };
    std::printf("%s, %d CUs: read stream over %zu MiB\n", prop.name, cus, total >> 20);
    for (int w : {8, 16, 32}) {
        bench("16 B/lane, 4 KB in flight", read_stream<false, 4>, w, 4);
        bench("16 B/lane, 8 KB in flight", read_stream<false, 8>, w, 8);
        bench("16 B/lane, 4 KB in flight, non-temporal", read_stream<true, 4>, w, 4);
        bench("16 B/lane, 8 KB in flight, non-temporal", read_stream<true, 8>, w, 8);
    }
    std::printf("{\"stream_ceiling_gbs\": %.1f, \"best\": \"%s\", \"bytes\": %zu}\n", best, best_name, total);
    return 0;
}
