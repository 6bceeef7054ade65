// Device-side TCA-BME encoder for gfx950: dense fp16 W in HBM -> bitmaps, offsets, values in HBM, bit-identical
// to the host encoder (csrc/SpMM_API.cuh:112-241 in the reference; spmspm_amd/csrc/encoder.cpp here).
//
// Byte work bound by HBM: W is read twice (8 KB per 64x64 group tile each time), the compressed arrays are
// written once.  Three kernels on the caller's stream:
//   encode_bitmaps   one wave per group tile; lane t owns 8x8 tile t (storage order 16*strip + 4*q + 2*j + i),
//                    reads its eight 16-byte rows (the 64 lanes of one load cover eight full 128-byte lines),
//                    builds the 64-bit mask (bit 8*r + c, non-zero test as the reference's half2float(v) != 0:
//                    -0.0 is dropped, NaN and subnormals are kept) and the wave writes the group tile's padded
//                    population to offsets[g + 1];
//   scan_*           in-place running sum of offsets[1..G], offsets[0] = 0 (three small kernels, no scratch);
//   encode_values    one wave per group tile again: a wave prefix sum of the tile populations gives every
//                    lane the position of its first value, the lanes compact their non-zeros into LDS in
//                    storage order, the run is padded with zeros to a multiple of eight and copied out with
//                    16-byte stores.
// The caller reads offsets[G] between the second and third kernel to size `values`.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>

#include "spmm_api.h"

namespace spmm_enc {

constexpr int kWavesPerWG = 4;
constexpr int kThreads    = 64 * kWavesPerWG;

template <int kCtrl, int kRowMask>
__device__ __forceinline__ int dpp_add(int x)
{
    return x + __builtin_amdgcn_update_dpp(0, x, kCtrl, kRowMask, 0xf, true);
}

__device__ __forceinline__ int wave_inclusive_scan(int x)
{
    x = dpp_add<0x111, 0xf>(x); // row_shr:1
    x = dpp_add<0x112, 0xf>(x); // row_shr:2
    x = dpp_add<0x114, 0xf>(x); // row_shr:4
    x = dpp_add<0x118, 0xf>(x); // row_shr:8
    x = dpp_add<0x142, 0xa>(x); // row_bcast:15 into rows 1 and 3
    x = dpp_add<0x143, 0xc>(x); // row_bcast:31 into rows 2 and 3
    return x;
}

typedef unsigned uintx4_t __attribute__((ext_vector_type(4)));

// The lane's 8x8 tile of group tile g: eight rows of eight halves, and its bitmap.
struct LaneTile {
    uint4    row[8];
    unsigned lo, hi;
};

__device__ __forceinline__ unsigned nonzero_bits(uint4 v) // bit c set when half c of the row is not +-0
{
    unsigned m = 0;
    m |= (v.x & 0x00007fffu) ? 1u : 0u;
    m |= (v.x & 0x7fff0000u) ? 2u : 0u;
    m |= (v.y & 0x00007fffu) ? 4u : 0u;
    m |= (v.y & 0x7fff0000u) ? 8u : 0u;
    m |= (v.z & 0x00007fffu) ? 16u : 0u;
    m |= (v.z & 0x7fff0000u) ? 32u : 0u;
    m |= (v.w & 0x00007fffu) ? 64u : 0u;
    m |= (v.w & 0x7fff0000u) ? 128u : 0u;
    return m;
}

__device__ __forceinline__ LaneTile load_lane_tile(const uint16_t* __restrict__ W, int K, int g, int lane)
{
    const int nkb = K >> 6;
    const int gm = g / nkb, gk = g - gm * nkb;
    const int strip = lane >> 4, q = (lane >> 2) & 3, j = (lane >> 1) & 1, i = lane & 1;
    const size_t r0 = (size_t)gm * 64 + strip * 16 + i * 8;
    const size_t c0 = (size_t)gk * 64 + q * 16 + j * 8;
    LaneTile     t;
    t.lo = t.hi = 0;
#pragma unroll
    for (int r = 0; r < 8; ++r)
        t.row[r] = __builtin_bit_cast(uint4, __builtin_nontemporal_load(reinterpret_cast<const uintx4_t*>(
            W + (r0 + r) * (size_t)K + c0))); // W streams through once per pass: 15 % faster with the hint in the
                                              // bitmap pass, 4 % in the value pass
#pragma unroll
    for (int r = 0; r < 4; ++r)
        t.lo |= nonzero_bits(t.row[r]) << (8 * r);
#pragma unroll
    for (int r = 4; r < 8; ++r)
        t.hi |= nonzero_bits(t.row[r]) << (8 * (r - 4));
    return t;
}

__global__ __launch_bounds__(kThreads) void encode_bitmaps(const uint16_t* __restrict__ W, int K, int G,
                                                           uint64_t* __restrict__ bitmaps, int* __restrict__ offsets)
{
    const int lane = threadIdx.x & 63;
    const int g    = blockIdx.x * kWavesPerWG + (threadIdx.x >> 6);
    if (g >= G)
        return;
    const LaneTile t = load_lane_tile(W, K, g, lane);
    bitmaps[(size_t)g * 64 + lane] = ((uint64_t)t.hi << 32) | t.lo;
    const int total = __builtin_amdgcn_readlane(wave_inclusive_scan(__builtin_popcount(t.lo) + __builtin_popcount(t.hi)), 63);
    if (lane == 0)
        offsets[g + 1] = (total + 7) & ~7; // the run is padded to a multiple of eight values
}

// offsets[0] = 0, offsets[1..G] <- running sum, in place and without scratch memory, in three small kernels
// over c[i] = offsets[1 + i]:
//   scan_blocks        every block of 1024 counts becomes its own inclusive sum (its last element = block total);
//   scan_block_totals  one workgroup turns the blocks' last elements into global inclusive sums;
//   add_block_prefix   block b >= 1 adds the last element of block b - 1 to all its elements but the last.
constexpr int kScanBlock = 1024;

// inclusive sum over the 256 threads of a workgroup (four waves); `red` is four ints of LDS
__device__ __forceinline__ int workgroup_inclusive_scan_256(int x, int* red)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int       inc  = wave_inclusive_scan(x);
    if (lane == 63)
        red[wave] = inc;
    __syncthreads();
    int before = 0;
    for (int w = 0; w < wave; ++w)
        before += red[w];
    __syncthreads();
    return inc + before;
}

__global__ __launch_bounds__(256) void scan_blocks(int* __restrict__ c, int G)
{
    __shared__ int buf[kScanBlock];
    __shared__ int red[4];
    const int base = blockIdx.x * kScanBlock;
    for (int i = threadIdx.x; i < kScanBlock; i += 256)
        buf[i] = base + i < G ? c[base + i] : 0;
    __syncthreads();
    int v[4], s = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        s += buf[4 * threadIdx.x + j];
        v[j] = s;
    }
    const int before = workgroup_inclusive_scan_256(s, red) - s;
#pragma unroll
    for (int j = 0; j < 4; ++j)
        buf[4 * threadIdx.x + j] = v[j] + before;
    __syncthreads();
    for (int i = threadIdx.x; i < kScanBlock; i += 256)
        if (base + i < G)
            c[base + i] = buf[i];
}

__global__ __launch_bounds__(256) void scan_block_totals(int* __restrict__ offsets, int G)
{
    __shared__ int red[4];
    int*      c  = offsets + 1;
    const int nb = (G + kScanBlock - 1) / kScanBlock;
    int       carry = 0;
    if (threadIdx.x == 0)
        offsets[0] = 0;
    for (int b0 = 0; b0 < nb; b0 += 256) { // 256 blocks (262144 group tiles) per round
        const int b    = b0 + threadIdx.x;
        const int last = ((b + 1) * kScanBlock < G ? (b + 1) * kScanBlock : G) - 1;
        const int x    = b < nb ? c[last] : 0;
        const int inc  = workgroup_inclusive_scan_256(x, red) + carry;
        if (b < nb)
            c[last] = inc;
        __shared__ int total;
        if (threadIdx.x == 255)
            total = inc;
        __syncthreads();
        carry = total;
        __syncthreads();
    }
}

__global__ __launch_bounds__(256) void add_block_prefix(int* __restrict__ c, int G)
{
    const int b    = blockIdx.x + 1;
    const int base = b * kScanBlock;
    const int end  = (base + kScanBlock < G ? base + kScanBlock : G) - 1; // the last element is already global
    const int add  = c[base - 1];
    for (int i = base + threadIdx.x; i < end; i += 256)
        c[i] += add;
}

__global__ __launch_bounds__(kThreads) void encode_values(const uint16_t* __restrict__ W, int K, int G,
                                                          const int* __restrict__ offsets,
                                                          uint16_t* __restrict__ values)
{
    __shared__ __attribute__((aligned(16))) uint16_t stage[kWavesPerWG][4096 + 8];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g    = blockIdx.x * kWavesPerWG + wave;
    if (g >= G)
        return;
    const LaneTile t   = load_lane_tile(W, K, g, lane);
    const int      pc  = __builtin_popcount(t.lo) + __builtin_popcount(t.hi);
    const int      inc = wave_inclusive_scan(pc);
    const int      total = __builtin_amdgcn_readlane(inc, 63);
    uint16_t*      out = stage[wave];
    int            p   = inc - pc; // position of this tile's first value in the group tile's run
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        const unsigned bits = ((r < 4 ? t.lo : t.hi) >> (8 * (r & 3))) & 0xffu;
        const unsigned d[4] = {t.row[r].x, t.row[r].y, t.row[r].z, t.row[r].w};
#pragma unroll
        for (int c = 0; c < 8; ++c)
            if (bits & (1u << c))
                out[p++] = (uint16_t)(d[c >> 1] >> (16 * (c & 1)));
    }
    const int padded = (total + 7) & ~7;
    if (lane < padded - total)
        out[total + lane] = 0;
    // the wave's own LDS writes are ordered before its reads below (lock step: no instruction; the fences hold the
    // compiler to that order although the accesses alias through casts)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int base = offsets[g];
    for (int i = lane; i < (padded >> 3); i += 64)
        reinterpret_cast<uint4*>(values + base)[i] = reinterpret_cast<const uint4*>(out)[i];
}

// ---- one pass over W ----------------------------------------------------------------------------------------------
// The two-call form reads W twice because a group tile's values cannot be placed before the populations of all
// earlier group tiles are known.  Here one kernel reads W once: a workgroup (four waves = four consecutive group
// tiles, taken in the order the workgroups start) builds its bitmaps and compacts its values into LDS, publishes the
// sum of its padded populations, and learns where its run begins by looking back over its predecessors' published
// sums (decoupled look-back: each predecessor shows either its own sum or, once it knows it, the sum of everything
// up to and including itself, so a workgroup never waits for more than the nearest predecessors still at work).
// Status words are 64 bits, {state, sum}, written and read whole with device-scope relaxed atomics: the word carries
// everything its reader needs, so no fence (which on this part would write back a whole L2) is involved.
// A workgroup only ever waits for workgroups that started before it and are therefore resident; the wait is bounded
// all the same, and a workgroup that gives up sets an error word and ends normally.
//
// Measured on 28672 x 7168 at 70 % sparsity: 189 us against 179 us for the two passes together (74 + 91 + 15 us),
// although only 561 MB cross the memory interface instead of 972 MB.  A workgroup's 32 KB of W are read in about the
// time one trip to another workgroup's status word takes, so the look-back is not hidden behind work: persistent
// workgroups that request their next rows of W before looking back (194 us), a window of 256 predecessors per trip
// instead of 64 (283-302 us: four times the words to wait for), one polling lane instead of 64, and chunks dealt
// round-robin without the ticket counter (220 us) all left it there or made it worse.  The call is kept for what it
// saves in traffic and for callers that want one launch; the two-call form remains the faster one.
constexpr unsigned kStateSum = 1, kStatePrefix = 2; // 0: nothing published yet
constexpr unsigned kErrSpin = 1, kErrCapacity = 2;
constexpr unsigned kSpinLimit = 1u << 16;

struct OnePassHeader {
    unsigned ticket, error, pad0, pad1;
};

__global__ __launch_bounds__(256) void zero_words(unsigned* p, size_t n)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n)
        p[i] = 0;
}

__device__ __forceinline__ unsigned long long status_load(const unsigned long long* p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void status_store(unsigned long long* p, unsigned state, unsigned sum)
{
    __hip_atomic_store(p, ((unsigned long long)state << 32) | sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__global__ __launch_bounds__(kThreads) void encode_onepass(const uint16_t* __restrict__ W, int K, int G,
                                                           uint64_t* __restrict__ bitmaps, int* __restrict__ offsets,
                                                           uint16_t* __restrict__ values, unsigned long long capacity,
                                                           OnePassHeader* __restrict__ head,
                                                           unsigned long long* __restrict__ status)
{
    __shared__ __attribute__((aligned(16))) uint16_t stage[kWavesPerWG][4096 + 8];
    __shared__ unsigned s_vid, s_excl;
    __shared__ int      s_count[kWavesPerWG];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (threadIdx.x == 0)
        s_vid = __hip_atomic_fetch_add(&head->ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    const unsigned vid    = s_vid; // position of this workgroup in start order = its chunk of four group tiles
    const long     g      = (long)vid * kWavesPerWG + wave;
    const bool     active = g < G;
    int            padded = 0;
    uint16_t*      out    = stage[wave];
    if (active) {
        const LaneTile t = load_lane_tile(W, K, (int)g, lane);
        bitmaps[(size_t)g * 64 + lane] = ((uint64_t)t.hi << 32) | t.lo;
        const int pc    = __builtin_popcount(t.lo) + __builtin_popcount(t.hi);
        const int inc   = wave_inclusive_scan(pc);
        const int total = __builtin_amdgcn_readlane(inc, 63);
        int       p     = inc - pc;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const unsigned bits = ((r < 4 ? t.lo : t.hi) >> (8 * (r & 3))) & 0xffu;
            const unsigned d[4] = {t.row[r].x, t.row[r].y, t.row[r].z, t.row[r].w};
#pragma unroll
            for (int c = 0; c < 8; ++c)
                if (bits & (1u << c))
                    out[p++] = (uint16_t)(d[c >> 1] >> (16 * (c & 1)));
        }
        padded = (total + 7) & ~7;
        if (lane < padded - total)
            out[total + lane] = 0;
    }
    if (lane == 0)
        s_count[wave] = padded;
    __syncthreads();
    unsigned agg = 0, before = 0;
#pragma unroll
    for (int w = 0; w < kWavesPerWG; ++w) {
        agg += (unsigned)s_count[w];
        before += w < wave ? (unsigned)s_count[w] : 0u;
    }
    if (wave == 0) {
        if (lane == 0)
            status_store(status + vid, vid == 0 ? kStatePrefix : kStateSum, agg);
        unsigned excl = 0;
        if (vid > 0) {
            long     j     = (long)vid - 1;
            unsigned spins = 0;
            for (;;) {
                const long               idx = j - lane; // lane 0 looks at the nearest predecessor
                // in front of the first chunk lies a prefix of zero
                const unsigned long long s   = idx >= 0 ? status_load(status + idx) : ((unsigned long long)kStatePrefix << 32);
                const unsigned           st  = (unsigned)(s >> 32);
                const unsigned long long inval = __ballot(st == 0), pref = __ballot(st == kStatePrefix);
                const int first_inval = inval ? __builtin_ctzll(inval) : 64;
                const int first_pref  = pref ? __builtin_ctzll(pref) : 64;
                if (first_inval < first_pref) { // a predecessor this side of the nearest prefix has not published yet
                    if (++spins > kSpinLimit) {
                        if (lane == 0)
                            __hip_atomic_fetch_or(&head->error, kErrSpin, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        break;
                    }
                    __builtin_amdgcn_s_sleep(2);
                    continue;
                }
                const int      upto    = first_pref < 64 ? first_pref : 63;
                const unsigned contrib = lane <= upto ? (unsigned)s : 0u;
                excl += (unsigned)__builtin_amdgcn_readlane(wave_inclusive_scan((int)contrib), 63);
                if (first_pref < 64)
                    break;
                j -= 64;
            }
            if (lane == 0)
                status_store(status + vid, kStatePrefix, excl + agg);
        }
        if (lane == 0)
            s_excl = excl;
    }
    __syncthreads();
    if (!active)
        return;
    const unsigned long long base = (unsigned long long)s_excl + before;
    if (lane == 0) {
        offsets[g + 1] = (int)(base + (unsigned)padded);
        if (g == 0)
            offsets[0] = 0;
    }
    if (base + (unsigned)padded > capacity) {
        if (lane == 0)
            __hip_atomic_fetch_or(&head->error, kErrCapacity, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return;
    }
    for (int i = lane; i < (padded >> 3); i += 64)
        reinterpret_cast<uint4*>(values + base)[i] = reinterpret_cast<const uint4*>(out)[i];
}

inline int check(int M, int K)
{
    if (M <= 0 || K <= 0 || M % 64 != 0 || K % 64 != 0) {
        std::printf("MM_Sparse_API Error: M (%d) and K (%d) must be positive multiples of 64!\n", M, K);
        std::fflush(stdout);
        return (int)hipErrorInvalidValue;
    }
    return 0;
}

} // namespace spmm_enc

extern "C" int SpMM_EncodeDevice_Bitmaps(hipStream_t stream, const void* W, int M, int K, uint64_t* bitmaps,
                                         int* offsets)
{
    if (int e = spmm_enc::check(M, K))
        return e;
    const int G = (M / 64) * (K / 64);
    (void)hipGetLastError();
    dim3 grid((unsigned)((G + spmm_enc::kWavesPerWG - 1) / spmm_enc::kWavesPerWG), 1, 1);
    hipLaunchKernelGGL(spmm_enc::encode_bitmaps, grid, dim3(spmm_enc::kThreads, 1, 1), 0, stream,
                       static_cast<const uint16_t*>(W), K, G, bitmaps, offsets);
    const int nb = (G + spmm_enc::kScanBlock - 1) / spmm_enc::kScanBlock;
    hipLaunchKernelGGL(spmm_enc::scan_blocks, dim3((unsigned)nb, 1, 1), dim3(256, 1, 1), 0, stream, offsets + 1, G);
    hipLaunchKernelGGL(spmm_enc::scan_block_totals, dim3(1, 1, 1), dim3(256, 1, 1), 0, stream, offsets, G);
    if (nb > 1)
        hipLaunchKernelGGL(spmm_enc::add_block_prefix, dim3((unsigned)(nb - 1), 1, 1), dim3(256, 1, 1), 0, stream,
                           offsets + 1, G);
    return (int)hipGetLastError();
}

extern "C" int SpMM_EncodeDevice_Values(hipStream_t stream, const void* W, int M, int K, const int* offsets,
                                        void* values)
{
    if (int e = spmm_enc::check(M, K))
        return e;
    const int G = (M / 64) * (K / 64);
    (void)hipGetLastError();
    dim3 grid((unsigned)((G + spmm_enc::kWavesPerWG - 1) / spmm_enc::kWavesPerWG), 1, 1);
    hipLaunchKernelGGL(spmm_enc::encode_values, grid, dim3(spmm_enc::kThreads, 1, 1), 0, stream,
                       static_cast<const uint16_t*>(W), K, G, offsets, static_cast<uint16_t*>(values));
    return (int)hipGetLastError();
}

extern "C" size_t SpMM_EncodeDevice_ScratchBytes(int M, int K)
{
    if (M <= 0 || K <= 0 || M % 64 != 0 || K % 64 != 0)
        return 0;
    const size_t G = (size_t)(M / 64) * (size_t)(K / 64);
    return sizeof(spmm_enc::OnePassHeader) + 8 * ((G + spmm_enc::kWavesPerWG - 1) / spmm_enc::kWavesPerWG);
}

extern "C" int SpMM_EncodeDevice_OnePass(hipStream_t stream, const void* W, int M, int K, uint64_t* bitmaps,
                                         int* offsets, void* values, size_t values_capacity, void* scratch)
{
    if (int e = spmm_enc::check(M, K))
        return e;
    if (scratch == nullptr || (reinterpret_cast<uintptr_t>(scratch) & 7) != 0)
        return (int)hipErrorInvalidValue;
    const int    G      = (M / 64) * (K / 64);
    const size_t chunks = ((size_t)G + spmm_enc::kWavesPerWG - 1) / spmm_enc::kWavesPerWG;
    const size_t words  = SpMM_EncodeDevice_ScratchBytes(M, K) / 4;
    (void)hipGetLastError();
    hipLaunchKernelGGL(spmm_enc::zero_words, dim3((unsigned)((words + 255) / 256), 1, 1), dim3(256, 1, 1), 0, stream,
                       static_cast<unsigned*>(scratch), words);
    auto* head   = static_cast<spmm_enc::OnePassHeader*>(scratch);
    auto* status = reinterpret_cast<unsigned long long*>(head + 1);
    hipLaunchKernelGGL(spmm_enc::encode_onepass, dim3((unsigned)chunks, 1, 1), dim3(spmm_enc::kThreads, 1, 1), 0, stream,
                       static_cast<const uint16_t*>(W), K, G, bitmaps, offsets, static_cast<uint16_t*>(values),
                       (unsigned long long)values_capacity, head, status);
    return (int)hipGetLastError();
}
