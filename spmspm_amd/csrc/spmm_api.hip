// Dispatcher, launcher and C ABI of the gfx950 bitmap SpMM.
// Replaces the host side of csrc/SpMM_API.cuh:21-110.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <dlfcn.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <tuple>
#include <vector>

#include "spmm_api.h"
#include "spmm_kernels.hiph"

namespace {

bool supported_n(int N)
{
    // The reference's switch (csrc/SpMM_API.cuh:60-96).
    return N == 8 || N == 16 || N == 32 || N == 64 || (N > 0 && N % 128 == 0);
}

int clamp_split_k(int split_k, int K)
{
    const int nkb = K / 64;
    if (split_k > nkb)
        split_k = nkb; // more batches than group-tile columns would leave empty batches
    return split_k < 1 ? 1 : split_k;
}

// K split of the wide kernel (N a multiple of 64, spmm_kernel_wide.hiph).  A workgroup covers 256 rows x 128 columns (64 at N = 64)
// x one K batch and two workgroups fit a CU, so the 512 slots are the unit: one round of at most 512 workgroups,
// each walking ceil(nkb / split) k blocks plus a start-up of about two.  Measured on OPT-66B FFN2 (9216 x 36864,
// N = 128): a workgroup alone on its CU takes 2.2 us per k block, two sharing a CU 3.45 us each (ratio 1.57);
// Split_K 7 / 12 / 14 / 16 -> 252 / 432 / 504 / 576 workgroups -> 177 / 151 / 141 / 177 us.  The partial slabs of a
// split are re-read from cache by the reduction, which adds little.  Over the 20 shapes on which the wide kernel was
// timed at every Split_K up to 32 (OPT-13B, 30B and 66B linears at N = 64 and 128) a sharing ratio of 1.4 and a
// tenth added to a launch that needs a second round pick the measured best split on all of them; with 1.57 and no
// addition three were off by 3 to 8 %.
int auto_split_k_wide(int M, int N, int K)
{
    const int    nkb  = K / 64;
    const long   base = (long)((M / 64 + 3) / 4) * (N / spmm::wide_tile_n(N));
    const double kSlots = 512.0, kAloneSlots = 256.0, kShared = 1.4, kSecondRound = 1.1, kStartup = 2.0;
    int          best = 1;
    double       best_c = 1e30;
    int          max_sk = nkb / 2 > 0 ? nkb / 2 : 1; // at least two k blocks per batch
    if (max_sk > 32)
        max_sk = 32;
    for (int sk = 1; sk <= max_sk; ++sk) {
        const double wgs    = (double)base * sk;
        const double rounds = (double)((long)((wgs + kSlots - 1) / kSlots));
        const double steps  = (double)((nkb + sk - 1) / sk) + kStartup;
        double       cost   = rounds * steps * (wgs > kAloneSlots ? kShared : 1.0) * (rounds > 1.0 ? kSecondRound : 1.0);
        if (sk > 1)
            cost += 1.0 + sk * ((double)M * N * 8.0) / 8e12 / 2.2e-6;
        if (cost < best_c - 1e-9) {
            best_c = cost;
            best   = sk;
        }
    }
    return best;
}

// Picks the K split from a small cost model (units: group tiles processed by the busiest CU), fitted to whole-call
// times (main kernel + reduction, back to back on one stream) of ten OPT-like shapes at Split_K 1..20, where its
// choice is within 4 % of the best measured split:
//   work     ceil(workgroups / 256) turns of (tiles per workgroup + a fixed start-up/epilogue cost);
//   fill     with fewer than two workgroups per CU the waves cannot hide each other's latencies;
//   partials a split adds the reduction kernel, and every batch writes and re-reads an fp32 slab of M*N.
int auto_split_k(int M, int N, int K)
{
    if (spmm::use_wide_kernel(M, N, K))
        return auto_split_k_wide(M, N, K);
    const int    nkb  = K / 64;
    const long   base = (long)(M / 64) * spmm::column_blocks(N);
    const double kCUs = 256.0, kStartupTiles = 2.0, kFillWGsPerCU = 2.0, kReductionTiles = 2.0, kTileBytes = 2000.0;
    if (base <= 0 || nkb <= 0)
        return 1;
    int    best    = 1;
    double best_c  = 1e30;
    int    max_sk  = nkb / 4 > 0 ? nkb / 4 : 1; // at least one group tile per wave and batch
    if (max_sk > 32)
        max_sk = 32;
    for (int sk = 1; sk <= max_sk; ++sk) {
        const double wgs   = (double)base * sk;
        const double turns = (double)((long)((wgs + kCUs - 1) / kCUs));
        const double tiles = (double)((nkb + sk - 1) / sk) + kStartupTiles;
        double       cost  = turns * tiles;
        const double per_cu = wgs / kCUs;
        if (per_cu < kFillWGsPerCU)
            cost *= kFillWGsPerCU / (per_cu < 0.25 ? 0.25 : per_cu);
        if (sk > 1)
            cost += kReductionTiles + sk * ((double)M * N * 8.0 / kCUs) / kTileBytes;
        if (cost < best_c - 1e-9) {
            best_c = cost;
            best   = sk;
        }
    }
    return best;
}

// Measured choices that take precedence over the cost model (the role of the reference's SplitKDict,
// end2end_inference/ft_tools/huggingface_opt_convert_Phase2.py:23, and of the SPLIT_K array of
// kernel_benchmark/run_all_main.sh:5): a table keyed by (M, N, K), filled by SpMM_SplitK_TableSet/SetMany or from a
// text file of "M N K Split_K" lines.  On first use a file is loaded: the one SPMM_SPLITK_TABLE names, or, when the
// variable is not set, the measured table shipped beside the library (../tuned/splitk_mi355x.txt from the
// library's own directory); SPMM_SPLITK_TABLE set to an empty string loads nothing.
// The table is an immutable snapshot behind a shared pointer: a reader takes a reference for the length of its
// look-up, a writer (rare: table set-up) copies the snapshot under the mutex, changes the copy and publishes it;
// a superseded snapshot is freed when its last reader lets go, so a process that retunes does not grow.
using SplitMap = std::map<std::tuple<int, int, int>, int>;
struct SplitTable {
    std::mutex                      lock;    // writers only
    std::shared_ptr<const SplitMap> current; // read and written with std::atomic_load / std::atomic_store
    std::atomic<bool>               env_checked{false};
};
SplitTable& split_table()
{
    static SplitTable t;
    return t;
}

// Calls `change` on a private copy of the table and publishes the copy.  Caller holds t.lock.
template <typename F>
void publish_locked(SplitTable& t, F change)
{
    std::shared_ptr<const SplitMap> cur = std::atomic_load_explicit(&t.current, std::memory_order_acquire);
    auto                            nxt = std::make_shared<SplitMap>(cur ? *cur : SplitMap());
    change(*nxt);
    std::atomic_store_explicit(&t.current, std::shared_ptr<const SplitMap>(std::move(nxt)), std::memory_order_release);
}

// returns the number of entries read, or -1 when the file cannot be opened, -2 on a malformed line (nothing is
// added then)
int load_split_table_locked(SplitTable& t, const char* path)
{
    std::FILE* f = std::fopen(path, "r");
    if (!f)
        return -1;
    char     line[256];
    SplitMap read;
    while (std::fgets(line, sizeof line, f)) {
        const char* p = line;
        while (*p == ' ' || *p == '\t')
            ++p;
        if (*p == '#' || *p == '\n' || *p == '\r' || *p == 0)
            continue;
        int m, nn, k, sk;
        if (std::sscanf(p, "%d %d %d %d", &m, &nn, &k, &sk) != 4 || m <= 0 || nn <= 0 || k <= 0 || sk < 1) {
            std::fclose(f);
            return -2;
        }
        read[std::make_tuple(m, nn, k)] = sk;
    }
    std::fclose(f);
    publish_locked(t, [&](SplitMap& m) {
        for (const auto& e : read)
            m[e.first] = e.second;
    });
    return (int)read.size();
}

// Path of the table shipped with the library: <directory of libSpMM_API.so>/../tuned/splitk_mi355x.txt.
std::string shipped_table_path()
{
    Dl_info info;
    if (!dladdr(reinterpret_cast<const void*>(&split_table), &info) || info.dli_fname == nullptr)
        return std::string();
    std::string       lib(info.dli_fname);
    const std::size_t slash = lib.find_last_of('/');
    const std::string dir   = slash == std::string::npos ? std::string(".") : lib.substr(0, slash);
    return dir + "/../tuned/splitk_mi355x.txt";
}

void check_env_table_once(SplitTable& t)
{
    if (t.env_checked.load(std::memory_order_acquire))
        return;
    std::lock_guard<std::mutex> g(t.lock);
    if (t.env_checked.load(std::memory_order_relaxed))
        return;
    if (const char* e = std::getenv("SPMM_SPLITK_TABLE")) {
        if (*e != 0) {
            const int n = load_split_table_locked(t, e);
            if (n < 0) {
                std::printf("MM_Sparse_API Warning: SPMM_SPLITK_TABLE=%s %s; using the built-in choice.\n", e,
                            n == -1 ? "cannot be opened" : "has a malformed line");
                std::fflush(stdout);
            }
        }
    } else {
        const std::string shipped = shipped_table_path();
        if (!shipped.empty())
            (void)load_split_table_locked(t, shipped.c_str()); // absent or unreadable: the cost model stands
    }
    t.env_checked.store(true, std::memory_order_release);
}

int split_k_for(int M, int N, int K)
{
    SplitTable& t = split_table();
    check_env_table_once(t);
    if (std::shared_ptr<const SplitMap> m = std::atomic_load_explicit(&t.current, std::memory_order_acquire)) {
        auto it = m->find(std::make_tuple(M, N, K));
        if (it != m->end())
            return clamp_split_k(it->second, K);
    }
    // the cost model's answer for the shape this thread asked about last is kept: a layer asks on every call
    thread_local int last_m = 0, last_n = 0, last_k = 0, last_sk = 0;
    if (M != last_m || N != last_n || K != last_k) {
        last_sk = clamp_split_k(auto_split_k(M, N, K), K);
        last_m = M, last_n = N, last_k = K;
    }
    return last_sk;
}

int check_shape(int M, int N, int K)
{
    if (!supported_n(N)) {
        std::printf("MM_Sparse_API Error: Unsupported N dimension %d!\n", N);
        std::fflush(stdout);
        return (int)hipErrorUnknown;
    }
    if (M <= 0 || K <= 0 || M % 64 != 0 || K % 64 != 0) {
        std::printf("MM_Sparse_API Error: M (%d) and K (%d) must be positive multiples of 64!\n", M, K);
        std::fflush(stdout);
        return (int)hipErrorInvalidValue;
    }
    if (M / 64 > 65535) { // row blocks are the z dimension of the launch grid
        std::printf("MM_Sparse_API Error: M (%d) exceeds 64 * 65535 rows!\n", M);
        std::fflush(stdout);
        return (int)hipErrorInvalidValue;
    }
    return 0;
}

// Optional timing hooks: the next SpMM call on this thread attaches these to its main kernel's dispatch.
thread_local hipEvent_t t_before_main = nullptr;
thread_local hipEvent_t t_after_main  = nullptr;

// An entry point that refuses its arguments before run() is reached drops the timing request too.
int refuse(int error)
{
    t_before_main = t_after_main = nullptr;
    return error;
}

int run(hipStream_t stream, const void* values, const uint64_t* bitmaps, const int* offsets, const void* X, void* C,
        int M, int N, int K, void* workspace, int split_k, bool fp32_partials, bool epilogue = false,
        const void* bias = nullptr, int act = 0)
{
    // the timing request belongs to this call whatever becomes of it
    hipEvent_t before = t_before_main, after = t_after_main;
    t_before_main = t_after_main = nullptr;
    if (int e = check_shape(M, N, K))
        return e;
    split_k = clamp_split_k(split_k, K);
    if ((split_k > 1 || epilogue) && workspace == nullptr) {
        std::printf("MM_Sparse_API Error: Split_K=%d needs a reduction workspace!\n", split_k);
        std::fflush(stdout);
        return (int)hipErrorInvalidValue;
    }
    // The kernels read and write 16 bytes at a time (8 for bitmaps): an address they cannot use is refused here, on the
    // host; on the device it would be a memory fault.
    const auto bad = [](const void* p, uintptr_t align) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) & (align - 1)) != 0; };
    if (bad(values, 16) || bad(bitmaps, 8) || bad(offsets, 4) || bad(X, 16) || bad(C, 16) ||
        (workspace != nullptr && bad(workspace, 16)) || (bias != nullptr && bad(bias, 2))) {
        std::printf("MM_Sparse_API Error: a null or misaligned device pointer (values, X, C and workspace: 16 bytes, "
                    "bitmaps: 8, offsets: 4)!\n");
        std::fflush(stdout);
        return (int)hipErrorInvalidValue;
    }
    hipError_t err = spmm::launch_spmm(stream, static_cast<const __half*>(values), bitmaps, offsets,
                                       static_cast<const __half*>(X), static_cast<__half*>(C), M, N, K, workspace,
                                       split_k, fp32_partials, before, after, epilogue);
    if (err != hipSuccess || (split_k == 1 && !epilogue))
        return (int)err;
    return (int)spmm::launch_reduction(stream, static_cast<__half*>(C), workspace, M, N, split_k, fp32_partials, bias,
                                       act);
}

} // namespace

extern "C" int SpMM_SplitK_Auto(int M, int N, int K)
{
    if (!supported_n(N) || M <= 0 || K <= 0 || M % 64 != 0 || K % 64 != 0)
        return 1;
    return split_k_for(M, N, K);
}

extern "C" int SpMM_SplitK_CostModel(int M, int N, int K)
{
    if (!supported_n(N) || M <= 0 || K <= 0 || M % 64 != 0 || K % 64 != 0)
        return 1;
    return clamp_split_k(auto_split_k(M, N, K), K);
}

extern "C" int SpMM_SplitK_TableSet(int M, int N, int K, int Split_K)
{
    if (!supported_n(N) || M <= 0 || K <= 0 || M % 64 != 0 || K % 64 != 0 || Split_K < 1)
        return (int)hipErrorInvalidValue;
    SplitTable& t = split_table();
    check_env_table_once(t); // the start-up file first: it must not undo this entry later
    std::lock_guard<std::mutex> g(t.lock);
    publish_locked(t, [&](SplitMap& m) { m[std::make_tuple(M, N, K)] = Split_K; });
    return 0;
}

extern "C" int SpMM_SplitK_TableSetMany(const int* entries, int count)
{
    if (count < 0 || (count > 0 && entries == nullptr))
        return (int)hipErrorInvalidValue;
    for (int i = 0; i < count; ++i) {
        const int M = entries[4 * i], N = entries[4 * i + 1], K = entries[4 * i + 2], sk = entries[4 * i + 3];
        if (!supported_n(N) || M <= 0 || K <= 0 || M % 64 != 0 || K % 64 != 0 || sk < 1)
            return (int)hipErrorInvalidValue; // nothing is recorded
    }
    SplitTable& t = split_table();
    check_env_table_once(t);
    std::lock_guard<std::mutex> g(t.lock);
    publish_locked(t, [&](SplitMap& m) {
        for (int i = 0; i < count; ++i)
            m[std::make_tuple(entries[4 * i], entries[4 * i + 1], entries[4 * i + 2])] = entries[4 * i + 3];
    });
    return 0;
}

extern "C" int SpMM_SplitK_TableLoad(const char* path)
{
    if (path == nullptr)
        return -1;
    SplitTable& t = split_table();
    check_env_table_once(t);
    std::lock_guard<std::mutex> g(t.lock);
    return load_split_table_locked(t, path);
}

extern "C" int SpMM_SplitK_TableSave(const char* path)
{
    if (path == nullptr)
        return -1;
    check_env_table_once(split_table());
    std::shared_ptr<const SplitMap> m = std::atomic_load_explicit(&split_table().current, std::memory_order_acquire);
    std::FILE*                      f = std::fopen(path, "w");
    if (!f)
        return -1;
    std::fprintf(f, "# M N K Split_K\n");
    int n = 0;
    if (m)
        for (const auto& e : *m) {
            std::fprintf(f, "%d %d %d %d\n", std::get<0>(e.first), std::get<1>(e.first), std::get<2>(e.first), e.second);
            ++n;
        }
    std::fclose(f);
    return n;
}

extern "C" void SpMM_SplitK_TableClear(void)
{
    SplitTable& t = split_table();
    check_env_table_once(t);
    std::lock_guard<std::mutex> g(t.lock);
    publish_locked(t, [](SplitMap& m) { m.clear(); });
}

extern "C" size_t SpMM_WorkspaceBytes(int M, int N, int K, int Split_K)
{
    if (!supported_n(N) || M <= 0 || K <= 0 || M % 64 != 0 || K % 64 != 0)
        return 0;
    int sk = Split_K <= 0 ? split_k_for(M, N, K) : clamp_split_k(Split_K, K);
    if (sk <= 1)
        return 0;
    return sizeof(float) * (size_t)M * (size_t)N * (size_t)sk;
}

extern "C" int SpMM_SplitK_API(hipStream_t stream, const void* values, const uint64_t* bitmaps, const int* offsets,
                               const void* X, void* C, int M, int N, int K, void* workspace, int Split_K)
{
    const int sk = Split_K <= 0 ? SpMM_SplitK_Auto(M, N, K) : Split_K; // 1 for a shape that run() will refuse
    return run(stream, values, bitmaps, offsets, X, C, M, N, K, workspace, sk, /*fp32_partials=*/true);
}

extern "C" int SpMM_SplitK_API_Sized(hipStream_t stream, const void* values, const uint64_t* bitmaps,
                                     const int* offsets, const void* X, void* C, int M, int N, int K, void* workspace,
                                     size_t workspace_bytes, int Split_K)
{
    if (int e = check_shape(M, N, K))
        return refuse(e);
    // resolved once: the size check and the launch see the same split
    const int sk = Split_K <= 0 ? split_k_for(M, N, K) : clamp_split_k(Split_K, K);
    if (sk > 1 && sizeof(float) * (size_t)M * (size_t)N * (size_t)sk > workspace_bytes) {
        std::printf("MM_Sparse_API Error: workspace of %zu bytes, Split_K %d needs %zu!\n", workspace_bytes, sk,
                    sizeof(float) * (size_t)M * (size_t)N * (size_t)sk);
        std::fflush(stdout);
        return refuse((int)hipErrorInvalidValue);
    }
    return run(stream, values, bitmaps, offsets, X, C, M, N, K, workspace, sk, /*fp32_partials=*/true);
}

extern "C" size_t SpMM_WorkspaceBytesBiasAct(int M, int N, int K, int Split_K)
{
    if (!supported_n(N) || M <= 0 || K <= 0 || M % 64 != 0 || K % 64 != 0)
        return 0;
    int sk = Split_K <= 0 ? split_k_for(M, N, K) : clamp_split_k(Split_K, K);
    return sizeof(float) * (size_t)M * (size_t)N * (size_t)sk; // one fp32 slab even for an unsplit K
}

extern "C" int SpMM_SplitK_API_BiasAct(hipStream_t stream, const void* values, const uint64_t* bitmaps,
                                       const int* offsets, const void* X, void* C, int M, int N, int K,
                                       void* workspace, int Split_K, const void* bias, int activation)
{
    if (int e = check_shape(M, N, K))
        return refuse(e);
    if (activation < 0 || activation > 2) {
        std::printf("MM_Sparse_API Error: unknown activation %d (0 none, 1 ReLU, 2 GELU)!\n", activation);
        std::fflush(stdout);
        return refuse((int)hipErrorInvalidValue);
    }
    int sk = Split_K <= 0 ? SpMM_SplitK_Auto(M, N, K) : Split_K;
    return run(stream, values, bitmaps, offsets, X, C, M, N, K, workspace, sk, /*fp32_partials=*/true,
               /*epilogue=*/true, bias, activation);
}

extern "C" int SpMM_SplitK_API_bitmap_v3(hipStream_t stream, const void* /*A*/, const void* Compressed_A,
                                         const int* TileOffsets, const int* /*TileOffsets_Median*/,
                                         const uint64_t* bitmap, const int* /*max_nnz_intile*/, const void* B,
                                         void* C, int M_Global, int N_Global, int K_Global,
                                         void* Reduction_Workspace, int Split_K)
{
    if (int e = check_shape(M_Global, N_Global, K_Global))
        return refuse(e);
    if (Split_K < 1) {
        std::printf("MM_Sparse_API Error: Split_K (%d) must be >= 1!\n", Split_K);
        std::fflush(stdout);
        return refuse((int)hipErrorInvalidValue);
    }
    return run(stream, Compressed_A, bitmap, TileOffsets, B, C, M_Global, N_Global, K_Global, Reduction_Workspace,
               Split_K, /*fp32_partials=*/false);
}

// ---- entry point that allocates nothing ---------------------------------------------------------------------
// The split-K partial sums live in a file-scope device array instead of a caller's workspace.  In host code the
// array's name is only a handle: its device address is looked up once per device and kept; every kernel argument
// uses that address.
namespace {

static __device__ __align__(256) unsigned char scratch[SPMM_NOALLOC_SCRATCH_BYTES];

constexpr int      kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];
std::mutex         g_scratch_lock;

// Device address of `scratch` on the current device, or nullptr (with *err set) when it cannot be found.
void* scratch_address(hipError_t* err)
{
    int dev = -1;
    *err    = hipGetDevice(&dev);
    if (*err != hipSuccess)
        return nullptr;
    if (dev < 0 || dev >= kMaxDevices) {
        *err = hipErrorInvalidDevice;
        return nullptr;
    }
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p != nullptr)
        return p;
    std::lock_guard<std::mutex> g(g_scratch_lock);
    p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p != nullptr)
        return p;
    void* found = nullptr;
    *err        = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
    if (*err != hipSuccess || found == nullptr) {
        if (*err == hipSuccess)
            *err = hipErrorNotFound;
        return nullptr;
    }
    g_scratch_ptr[dev].store(found, std::memory_order_release);
    return found;
}

} // namespace

extern "C" int SpMM_SplitK_API_NoAlloc(hipStream_t stream, const void* values, const uint64_t* bitmaps,
                                       const int* offsets, const void* X, void* C, int M, int N, int K, int Split_K)
{
    if (int e = check_shape(M, N, K))
        return refuse(e);
    int          sk   = Split_K <= 0 ? split_k_for(M, N, K) : clamp_split_k(Split_K, K);
    const size_t slab = sizeof(float) * (size_t)M * (size_t)N;
    if (Split_K <= 0 && sk > 1 && slab * (size_t)sk > (size_t)SPMM_NOALLOC_SCRATCH_BYTES) {
        // the library's own choice gives way to the largest split whose partial sums fit; an unsplit K needs none
        sk = (int)((size_t)SPMM_NOALLOC_SCRATCH_BYTES / slab);
        if (sk < 2)
            sk = 1;
    }
    const size_t need = sk > 1 ? slab * (size_t)sk : 0;
    if (need > (size_t)SPMM_NOALLOC_SCRATCH_BYTES) {
        std::printf("MM_Sparse_API Error: M=%d N=%d Split_K=%d needs %zu bytes of partial sums; "
                    "SpMM_SplitK_API_NoAlloc holds at most %zu!\n",
                    M, N, sk, need, (size_t)SPMM_NOALLOC_SCRATCH_BYTES);
        std::fflush(stdout);
        return refuse((int)hipErrorInvalidValue);
    }
    void* ws = nullptr;
    if (sk > 1) {
        hipError_t err = hipSuccess;
        ws             = scratch_address(&err);
        if (ws == nullptr) {
            std::printf("MM_Sparse_API Error: the library's scratch array was not found on this device (%s)!\n",
                        hipGetErrorString(err));
            std::fflush(stdout);
            return refuse((int)err);
        }
    }
    return run(stream, values, bitmaps, offsets, X, C, M, N, K, ws, sk, /*fp32_partials=*/true);
}

extern "C" int SpMM_SplitK_AutoNoAlloc(int M, int N, int K)
{
    if (!supported_n(N) || M <= 0 || K <= 0 || M % 64 != 0 || K % 64 != 0)
        return 1;
    int          sk   = split_k_for(M, N, K);
    const size_t slab = sizeof(float) * (size_t)M * (size_t)N;
    if (sk > 1 && slab * (size_t)sk > (size_t)SPMM_NOALLOC_SCRATCH_BYTES) {
        sk = (int)((size_t)SPMM_NOALLOC_SCRATCH_BYTES / slab);
        if (sk < 2)
            sk = 1;
    }
    return sk;
}

// ---- the six weight files -> device arrays (the consumer side of Our_GenSparseMatrixBinFile) -------------------
extern "C" void SpMM_FreeWeights(void* values_d, int* offsets_d, int* median_d, uint64_t* bitmaps_d, int* max_nnz_d)
{
    void* all[5] = {values_d, offsets_d, median_d, bitmaps_d, max_nnz_d};
    for (void* p : all)
        if (p != nullptr)
            (void)hipFree(p);
}

extern "C" int SpMM_LoadWeightFiles(const char* Compressed_ValFileName, const char* TileOffsets_globalFileName,
                                    const char* TileOffsets_medianFileName, const char* bitmapFileName,
                                    const char* max_nnz_intileFileName, const char* OutputSizesFileName, int M, int K,
                                    void** values_d, int** offsets_d, int** median_d, uint64_t** bitmaps_d,
                                    int** max_nnz_d, int* val_count)
{
    if (values_d == nullptr || offsets_d == nullptr || bitmaps_d == nullptr)
        return -4;
    uint16_t* vals   = nullptr;
    int *     global = nullptr, *median = nullptr;
    uint64_t* bitmap = nullptr;
    int       max_nnz = 0, count = 0;
    const int G = SpMM_ReadWeightFiles(Compressed_ValFileName, TileOffsets_globalFileName, TileOffsets_medianFileName,
                                       bitmapFileName, max_nnz_intileFileName, OutputSizesFileName, M, K, &vals,
                                       &global, &median, &bitmap, &max_nnz, &count);
    if (G < 0)
        return G;
    void *    dv = nullptr, *dg = nullptr, *dm = nullptr, *db = nullptr, *dn = nullptr;
    const size_t bytes_v = sizeof(uint16_t) * (size_t)count, bytes_g = sizeof(int) * ((size_t)G + 1),
                 bytes_m = sizeof(int) * 4 * (size_t)G, bytes_b = sizeof(uint64_t) * 64 * (size_t)G;
    hipError_t err = hipMalloc(&dv, bytes_v ? bytes_v : 16); // an all-zero matrix still gets a valid pointer
    if (err == hipSuccess) err = hipMalloc(&dg, bytes_g);
    if (err == hipSuccess) err = hipMalloc(&db, bytes_b);
    if (err == hipSuccess && median_d != nullptr) err = hipMalloc(&dm, bytes_m);
    if (err == hipSuccess && max_nnz_d != nullptr) err = hipMalloc(&dn, sizeof(int));
    if (err == hipSuccess && bytes_v) err = hipMemcpy(dv, vals, bytes_v, hipMemcpyHostToDevice);
    if (err == hipSuccess) err = hipMemcpy(dg, global, bytes_g, hipMemcpyHostToDevice);
    if (err == hipSuccess) err = hipMemcpy(db, bitmap, bytes_b, hipMemcpyHostToDevice);
    if (err == hipSuccess && dm != nullptr) err = hipMemcpy(dm, median, bytes_m, hipMemcpyHostToDevice);
    if (err == hipSuccess && dn != nullptr) err = hipMemcpy(dn, &max_nnz, sizeof(int), hipMemcpyHostToDevice);
    std::free(vals), std::free(global), std::free(median), std::free(bitmap);
    if (err != hipSuccess) {
        std::printf("MM_Sparse_API Error: SpMM_LoadWeightFiles: %s!\n", hipGetErrorString(err));
        std::fflush(stdout);
        SpMM_FreeWeights(dv, static_cast<int*>(dg), static_cast<int*>(dm), static_cast<uint64_t*>(db),
                         static_cast<int*>(dn));
        return -5;
    }
    *values_d  = dv;
    *offsets_d = static_cast<int*>(dg);
    *bitmaps_d = static_cast<uint64_t*>(db);
    if (median_d != nullptr)
        *median_d = static_cast<int*>(dm);
    if (max_nnz_d != nullptr)
        *max_nnz_d = static_cast<int*>(dn);
    if (val_count != nullptr)
        *val_count = count;
    return G;
}

extern "C" void SpMM_TimeNextCall(hipEvent_t before_main, hipEvent_t after_main)
{
    t_before_main = before_main;
    t_after_main  = after_main;
}

// ---- shader clock probe ---------------------------------------------------------------------------------------
// One wave spins for about `spin_us` microseconds of the constant 100 MHz counter (s_memrealtime) and reports how
// far the shader-clock counter (s_memtime) advanced meanwhile.  Launched on a second stream while SpMM calls run, it
// reads the clock the kernels actually run at, which is what a kernel bound inside the CU follows.
namespace {
__global__ __launch_bounds__(64) void shader_clock_probe(unsigned long long* out, unsigned spin_ticks)
{
    const unsigned long long r0 = __builtin_amdgcn_s_memrealtime(), c0 = __builtin_readcyclecounter();
    unsigned long long       r1 = r0;
    for (unsigned i = 0; i < (1u << 22) && r1 - r0 < spin_ticks; ++i) { // bounded: every wave reaches the end
        __builtin_amdgcn_s_sleep(8);
        r1 = __builtin_amdgcn_s_memrealtime();
    }
    const unsigned long long c1 = __builtin_readcyclecounter();
    if (threadIdx.x == 0) {
        out[0] = c1 - c0;
        out[1] = r1 - r0;
    }
}
} // namespace

extern "C" int SpMM_ShaderClockProbe(hipStream_t stream, unsigned long long* ticks_d, int spin_us)
{
    if (ticks_d == nullptr || spin_us <= 0 || spin_us > 100000)
        return (int)hipErrorInvalidValue;
    return (int)spmm::launch_kernel(shader_clock_probe, dim3(1, 1, 1), dim3(64, 1, 1), stream, nullptr, nullptr,
                                    ticks_d, (unsigned)spin_us * 100u);
}

#ifdef SPMM_KEEP_VARIANTS
// Test build only (not in the header): selects the comparison kernel for the calls that follow.
extern "C" void SpMM_Debug_SetKernelVariant(int variant)
{
    spmm::kernel_variant() = variant;
}
#endif

extern "C" const char* SpMM_KernelName(int M, int N, int K, int Split_K)
{
    if (!supported_n(N) || M <= 0 || K <= 0 || M % 64 != 0 || K % 64 != 0)
        return nullptr;
    thread_local char name[64];
    const int         sk   = Split_K <= 0 ? split_k_for(M, N, K) : clamp_split_k(Split_K, K);
    const char*       fp32 = sk > 1 ? "true" : "false"; // SpMM_SplitK_API: partial sums in fp32 whenever K is split
    if (spmm::use_wide_kernel(M, N, K))
        std::snprintf(name, sizeof name, "spmm::spmm_bitmap_wide<%d, %s>", spmm::wide_tile_n(N) / 16, fp32);
    else
        std::snprintf(name, sizeof name, "spmm::spmm_bitmap_rows<%d, %s>", spmm::tile_n(N) / 16, fp32);
    return name;
}

extern "C" const char* SpMM_Version(void)
{
    return "spmm-gfx950 0.1";
}
