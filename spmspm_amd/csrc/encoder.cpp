// Host encoder: dense row-major fp16 W[M][K] -> TCA-BME arrays.
//
// Produces, bit for bit, what the reference's InitSparseMatrixA_bitmap
// produces (csrc/SpMM_API.cuh:112-241) but is organised differently: the
// reference walks the matrix once on one thread, appending values as it goes;
// here the 64-row blocks are independent work items.  Pass 1 builds every
// bitmap, per-tile count, strip offset and padded group-tile count in
// parallel; a serial exclusive prefix sum turns the counts into
// TileOffsets_global; pass 2 writes each group tile's values at its final
// position, again in parallel.  Only host code lives in this file.
#include <algorithm>
#include <atomic>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <thread>
#include <vector>

#include <hip/hip_fp16.h>

#include "spmm_api.h"

namespace {

// Storage order of the 16 8x8 tiles of one 16x64 strip: column pairs left to
// right, and inside a pair the 2x2 quad column-major
// (csrc/SpMM_API.cuh:167-173).  local index lt = 4*q + 2*j + i.
inline void tile_origin(int lt, int& row, int& col)
{
    row = (lt & 1) * 8;
    col = ((lt >> 2) & 3) * 16 + ((lt >> 1) & 1) * 8;
}

// A half is kept iff its float value != 0.0f (csrc/SpMM_API.cuh:189): both
// zeros have all magnitude bits clear; NaN and subnormals do not.
inline bool kept(uint16_t h)
{
    return (h & 0x7fffu) != 0;
}

// Bitmap of the 8x8 tile whose top-left element is `p` (row stride `ld`).
inline uint64_t tile_bitmap(const uint16_t* p, size_t ld)
{
    uint64_t bm = 0;
    for (int r = 0; r < 8; ++r) {
        const uint16_t* row = p + r * ld;
        unsigned        byte = 0;
        for (int c = 0; c < 8; ++c)
            byte |= (unsigned)kept(row[c]) << c;
        bm |= (uint64_t)byte << (8 * r);
    }
    return bm;
}

unsigned worker_count(size_t items)
{
    unsigned n = std::thread::hardware_concurrency();
    if (const char* e = std::getenv("SPMM_ENCODER_THREADS")) {
        int v = std::atoi(e);
        if (v > 0)
            n = (unsigned)v;
    }
    if (n == 0)
        n = 1;
    return (unsigned)std::min<size_t>(n, std::max<size_t>(items, 1));
}

template <class F>
void parallel_rows(int count, F&& body)
{
    unsigned nthreads = worker_count((size_t)count);
    if (nthreads <= 1) {
        for (int i = 0; i < count; ++i)
            body(i);
        return;
    }
    std::atomic<int>         next{0};
    std::vector<std::thread> pool;
    pool.reserve(nthreads);
    for (unsigned t = 0; t < nthreads; ++t)
        pool.emplace_back([&] {
            for (int i = next.fetch_add(1); i < count; i = next.fetch_add(1))
                body(i);
        });
    for (auto& th : pool)
        th.join();
}

int encode(const uint16_t* A, int M, int K, uint16_t** vals_out, int** cnt_out, int** median_out, int** global_out,
           uint64_t** bitmap_out, int* max_nnz_out)
{
    const int    gm_n = M / 64, gk_n = K / 64;
    const int    G = gm_n * gk_n;
    const size_t T = (size_t)(M / 8) * (size_t)(K / 8);
    const size_t ld = (size_t)K;

    // The reference sizes the per-tile arrays by (M/8)*(K/8) (:124,:136,:139)
    // and the strip-offset array generously (:137); only the first 64*G / 4*G
    // entries are ever written.  Keep the per-tile sizes, allocate 4*G strips.
    int*      cnt    = (int*)std::malloc(std::max<size_t>(T, 1) * sizeof(int));
    int*      median = (int*)std::malloc(std::max<size_t>((size_t)G * 4, 1) * sizeof(int));
    int*      global = (int*)std::malloc(((size_t)G + 1) * sizeof(int));
    uint64_t* bitmap = (uint64_t*)std::malloc(std::max<size_t>(T, 1) * sizeof(uint64_t));
    if (!cnt || !median || !global || !bitmap) {
        std::free(cnt), std::free(median), std::free(global), std::free(bitmap);
        return -1;
    }
    if (T > (size_t)G * 64) { // tail tiles outside whole group tiles: defined contents instead of garbage
        std::memset(cnt + (size_t)G * 64, 0, (T - (size_t)G * 64) * sizeof(int));
        std::memset(bitmap + (size_t)G * 64, 0, (T - (size_t)G * 64) * sizeof(uint64_t));
    }

    // Pass 1: bitmaps, counts, strip offsets, padded group counts (in global[g+1]).
    global[0] = 0;
    parallel_rows(gm_n, [&](int gm) {
        for (int gk = 0; gk < gk_n; ++gk) {
            const size_t    g    = (size_t)gm * gk_n + gk;
            const uint16_t* base = A + (size_t)gm * 64 * ld + (size_t)gk * 64;
            int             run  = 0;
            for (int strip = 0; strip < 4; ++strip) {
                median[g * 4 + strip] = run;
                for (int lt = 0; lt < 16; ++lt) {
                    int r0, c0;
                    tile_origin(lt, r0, c0);
                    uint64_t bm = tile_bitmap(base + (size_t)(strip * 16 + r0) * ld + c0, ld);
                    int      c  = __builtin_popcountll(bm);
                    bitmap[g * 64 + strip * 16 + lt] = bm;
                    cnt[g * 64 + strip * 16 + lt]    = c;
                    run += c;
                }
            }
            global[g + 1] = (run + 7) & ~7; // zero-padded to a multiple of 8 (:216-220)
        }
    });

    int max_nnz = 0;
    for (int g = 0; g < G; ++g) {
        max_nnz = std::max(max_nnz, global[g + 1]);
        global[g + 1] += global[g];
    }
    const size_t total = (size_t)global[G];

    uint16_t* vals = (uint16_t*)std::malloc(std::max<size_t>(total, 1) * sizeof(uint16_t));
    if (!vals) {
        std::free(cnt), std::free(median), std::free(global), std::free(bitmap);
        return -1;
    }

    // Pass 2: compact values in bit order, tile after tile, then the zero padding.
    parallel_rows(gm_n, [&](int gm) {
        for (int gk = 0; gk < gk_n; ++gk) {
            const size_t    g    = (size_t)gm * gk_n + gk;
            const uint16_t* base = A + (size_t)gm * 64 * ld + (size_t)gk * 64;
            uint16_t*       out  = vals + global[g];
            uint16_t* const end  = vals + global[g + 1];
            for (int t = 0; t < 64; ++t) {
                int r0, c0;
                tile_origin(t & 15, r0, c0);
                const uint16_t* p  = base + (size_t)((t >> 4) * 16 + r0) * ld + c0;
                uint64_t        bm = bitmap[g * 64 + t];
                while (bm) {
                    int b  = __builtin_ctzll(bm);
                    *out++ = p[(size_t)(b >> 3) * ld + (b & 7)];
                    bm &= bm - 1;
                }
            }
            while (out < end)
                *out++ = 0; // +0.0
        }
    });

    *vals_out    = vals;
    *cnt_out     = cnt;
    *median_out  = median;
    *global_out  = global;
    *bitmap_out  = bitmap;
    *max_nnz_out = max_nnz;
    return G;
}

bool reference_tiling(int tile_M, int tile_M_median, int tile_M_global, int tile_K, int tile_K_median,
                      int tile_K_global)
{
    return tile_M == 8 && tile_M_median == 16 && tile_M_global == 64 && tile_K == 8 && tile_K_median == 64 &&
           tile_K_global == 64;
}

} // namespace

extern "C" int InitSparseMatrixA_bitmap(uint16_t* A_h, int M, int K, int tile_M, int tile_M_median,
                                        int tile_M_global, int tile_K, int tile_K_median, int tile_K_global,
                                        uint16_t** Compressed_Val, int** TileOffsets, int** TileOffsets_median,
                                        int** TileOffsets_global, uint64_t** bitmap, int* max_nnz_count)
{
    if (!reference_tiling(tile_M, tile_M_median, tile_M_global, tile_K, tile_K_median, tile_K_global))
        return -2;
    if (M < 0 || K < 0 || !max_nnz_count)
        return -2;
    return encode(A_h, M, K, Compressed_Val, TileOffsets, TileOffsets_median, TileOffsets_global, bitmap,
                  max_nnz_count);
}

// C++ overload carrying the reference's mangled name (csrc/SpMM_API.cuh:112-120).
int InitSparseMatrixA_bitmap(__half* A_h, int M, int K, int tile_M, int tile_M_median, int tile_M_global, int tile_K,
                             int tile_K_median, int tile_K_global, __half** Compressed_Val, int** TileOffsets,
                             int** TileOffsets_median, int** TileOffsets_global, uint64_t** bitmap,
                             int& max_nnz_count)
{
    static_assert(sizeof(__half) == sizeof(uint16_t), "fp16 is two bytes");
    return InitSparseMatrixA_bitmap(reinterpret_cast<uint16_t*>(A_h), M, K, tile_M, tile_M_median, tile_M_global,
                                    tile_K, tile_K_median, tile_K_global,
                                    reinterpret_cast<uint16_t**>(Compressed_Val), TileOffsets, TileOffsets_median,
                                    TileOffsets_global, bitmap, &max_nnz_count);
}

// File-to-file wrapper (csrc/SpMM_API.cuh:243-320): same six output files,
// same contents, same messages and exit(-1) on I/O failure.
extern "C" void Our_GenSparseMatrixBinFile(char* DenseMatrixFileName, int M, int K, char* Compressed_ValFileName,
                                           char* bitmap_TileOffsets_globalFileName,
                                           char* bitmap_TileOffsets_medianFileName, char* bitmapFileName,
                                           char* max_nnz_intileFileName, char* OutputSizesFileName)
{
    const size_t          want = sizeof(uint16_t) * (size_t)M * (size_t)K;
    std::vector<uint16_t> dense((size_t)M * (size_t)K);
    std::ifstream         in(DenseMatrixFileName, std::ios::in | std::ios::binary);
    if (!in.is_open()) {
        std::printf("file %s cannot be opened, loadDataArrayFromBin fails. \n", DenseMatrixFileName);
        std::exit(-1);
    }
    in.read(reinterpret_cast<char*>(dense.data()), (std::streamsize)want);
    const size_t got = (size_t)in.gcount();
    if (got != want) {
        std::printf("file %s only has %ld, but request %ld, loading DenseMatrix fails! \n", DenseMatrixFileName,
                    (long)got, (long)want);
        std::exit(-1);
    }
    in.close();

    uint16_t* vals   = nullptr;
    int *     cnt    = nullptr, *median = nullptr, *global = nullptr;
    uint64_t* bitmap = nullptr;
    int       max_nnz = 0;
    int G = encode(dense.data(), M, K, &vals, &cnt, &median, &global, &bitmap, &max_nnz);
    if (G < 0) {
        std::printf("Our_GenSparseMatrixBinFile() ERROR: out of memory.\n");
        std::exit(-1);
    }
    int num_ltiles = G * 64, num_mtiles = G * 4, num_gtiles_p1 = G + 1;
    int val_count  = global[G];
    if (max_nnz % 64 != 0)
        max_nnz = ((max_nnz / 64) + 1) * 64; // :284-286
    std::printf("num_global_tiles: %d, bitmap v3 NNZ: %d, max_nnz_intilev3: %d \n", G, val_count, max_nnz);

    std::ofstream f_sizes(OutputSizesFileName, std::ios::out | std::ios::binary);
    std::ofstream f_vals(Compressed_ValFileName, std::ios::out | std::ios::binary);
    std::ofstream f_global(bitmap_TileOffsets_globalFileName, std::ios::out | std::ios::binary);
    std::ofstream f_median(bitmap_TileOffsets_medianFileName, std::ios::out | std::ios::binary);
    std::ofstream f_bitmap(bitmapFileName, std::ios::out | std::ios::binary);
    std::ofstream f_nnz(max_nnz_intileFileName, std::ios::out | std::ios::binary);
    if (!f_sizes.is_open() || !f_vals.is_open() || !f_global.is_open() || !f_median.is_open() ||
        !f_bitmap.is_open() || !f_nnz.is_open()) {
        std::printf("Our_GenSparseMatrixBinFile() ERROR: file %s, %s, %s, %s, %s or %s cannot be opened or creaetd. \n",
                    OutputSizesFileName, Compressed_ValFileName, bitmap_TileOffsets_globalFileName,
                    bitmap_TileOffsets_medianFileName, bitmapFileName, max_nnz_intileFileName);
        std::exit(-1);
    }
    // sizes: {val_count, G+1, 4G, 64G} (:304-308)
    f_sizes.write(reinterpret_cast<char*>(&val_count), sizeof(int));
    f_sizes.write(reinterpret_cast<char*>(&num_gtiles_p1), sizeof(int));
    f_sizes.write(reinterpret_cast<char*>(&num_mtiles), sizeof(int));
    f_sizes.write(reinterpret_cast<char*>(&num_ltiles), sizeof(int));
    f_vals.write(reinterpret_cast<char*>(vals), (std::streamsize)(sizeof(uint16_t) * (size_t)val_count));
    f_global.write(reinterpret_cast<char*>(global), (std::streamsize)(sizeof(int) * (size_t)num_gtiles_p1));
    f_median.write(reinterpret_cast<char*>(median), (std::streamsize)(sizeof(int) * (size_t)num_mtiles));
    f_bitmap.write(reinterpret_cast<char*>(bitmap), (std::streamsize)(sizeof(uint64_t) * (size_t)num_ltiles));
    f_nnz.write(reinterpret_cast<char*>(&max_nnz), sizeof(int));
    std::free(vals), std::free(cnt), std::free(median), std::free(global), std::free(bitmap);
}

// Reader of those six files (the consumer side: third_party/ft_spinfer.patch:2335-2357 loads them with
// loadDataArrayFromBin into arrays sized from the model's configuration).  Unlike the writer it reports failure to
// its caller instead of ending the process.
namespace {

// the whole file as `count` elements of `size` bytes, malloc'd; nullptr when it is missing or has another length
void* read_exact(const char* path, size_t size, size_t count)
{
    std::FILE* f = std::fopen(path, "rb");
    if (!f)
        return nullptr;
    void*  buf = std::malloc(size * count ? size * count : 1);
    size_t got = buf ? std::fread(buf, size, count, f) : 0;
    char   extra;
    const bool longer = std::fread(&extra, 1, 1, f) == 1;
    std::fclose(f);
    if (buf == nullptr || got != count || longer) {
        std::free(buf);
        return nullptr;
    }
    return buf;
}

} // namespace

extern "C" int SpMM_ReadWeightFiles(const char* Compressed_ValFileName, const char* TileOffsets_globalFileName,
                                    const char* TileOffsets_medianFileName, const char* bitmapFileName,
                                    const char* max_nnz_intileFileName, const char* OutputSizesFileName, int M, int K,
                                    uint16_t** Compressed_Val, int** TileOffsets_global, int** TileOffsets_median,
                                    uint64_t** bitmap, int* max_nnz_intile, int* val_count)
{
    if (!Compressed_ValFileName || !TileOffsets_globalFileName || !TileOffsets_medianFileName || !bitmapFileName ||
        !max_nnz_intileFileName || !OutputSizesFileName || !Compressed_Val || !TileOffsets_global || !bitmap)
        return -4;
    if (M <= 0 || K <= 0 || M % 64 != 0 || K % 64 != 0)
        return -2;
    int* sizes = static_cast<int*>(read_exact(OutputSizesFileName, sizeof(int), 4));
    if (sizes == nullptr)
        return -1;
    const long G = (long)(M / 64) * (K / 64);
    const int  count = sizes[0];
    const bool fits  = count >= 0 && count % 8 == 0 && sizes[1] == G + 1 && sizes[2] == 4 * G && sizes[3] == 64 * G;
    std::free(sizes);
    if (!fits)
        return -2;
    uint16_t* vals   = static_cast<uint16_t*>(read_exact(Compressed_ValFileName, sizeof(uint16_t), (size_t)count));
    int*      global = static_cast<int*>(read_exact(TileOffsets_globalFileName, sizeof(int), (size_t)G + 1));
    int*      median = static_cast<int*>(read_exact(TileOffsets_medianFileName, sizeof(int), 4 * (size_t)G));
    uint64_t* bm     = static_cast<uint64_t*>(read_exact(bitmapFileName, sizeof(uint64_t), 64 * (size_t)G));
    int*      nnz    = static_cast<int*>(read_exact(max_nnz_intileFileName, sizeof(int), 1));
    int       rc     = (int)G;
    if (!vals || !global || !median || !bm || !nnz)
        rc = -1;
    else if (global[0] != 0 || global[G] != count)
        rc = -2; // the offsets do not describe the values file
    else
        for (long g = 0; g < G && rc >= 0; ++g)
            if (global[g + 1] < global[g] || (global[g + 1] - global[g]) % 8 != 0 || global[g + 1] - global[g] > 4096)
                rc = -2;
    if (rc < 0) {
        std::free(vals), std::free(global), std::free(median), std::free(bm), std::free(nnz);
        return rc;
    }
    *Compressed_Val     = vals;
    *TileOffsets_global = global;
    *bitmap             = bm;
    if (TileOffsets_median != nullptr)
        *TileOffsets_median = median;
    else
        std::free(median);
    if (max_nnz_intile != nullptr)
        *max_nnz_intile = *nnz;
    std::free(nnz);
    if (val_count != nullptr)
        *val_count = count;
    return rc;
}
