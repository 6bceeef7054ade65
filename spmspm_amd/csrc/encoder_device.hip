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
// A second form, further down, reads W once in a single kernel (for a caller that can give `values` room before the
// number of values is known).
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
// earlier group tiles are known.  Here one kernel reads W once.  A chunk is kOnePassWaves consecutive group tiles, one
// per wave of a workgroup; workgroups take chunks in the order they start (a ticket counter), so a workgroup only
// ever waits for workgroups that are resident.  A workgroup
//   1. reads its rows of W, writes the bitmaps and publishes the chunk's padded population (`status`, one 64-bit word
//      per chunk, {1, sum});
//   2. requests the words that tell it where its run begins, and compacts its values into LDS while they travel;
//   3. start = its predecessors inside its block of 64 chunks (one status word per lane) + the blocks in front of its
//      block (`bword`, one word per block and lane, 64 blocks per trip) back to the nearest one that shows the sum of
//      everything up to its end.  The last chunk of a block speaks for the block: once its 63 predecessors have
//      published it writes {1, the block's sum}, and once it knows its own start {2, the sum up to the block's end}.
//      Words that are not there yet are polled (bounded);
//   4. writes the offsets and copies the runs from LDS to `values`.
// Every word carries all its reader needs and is written and read whole with relaxed device-scope atomics: no fence
// (which on this part would write back a whole L2) is involved.  A wave's LDS stage holds kStage values: a group tile
// up to half full is compacted in one go, a fuller one in two halves (the tile stays in registers meanwhile); with
// the full 4096 a CU would hold one workgroup instead of two.
//
// Measured on 28672 x 7168 at 70 % sparsity (MI355X; the two calls take 179 us, a kernel that only reads W 65 us):
//   16 group tiles per chunk 110 us, 8: 128 us, 4: 184 us.  The ticket decides: an atomic on one address completes
//   every 14.6 ns on this device (time stamps taken inside the kernel: the first 2048 tickets arrive over 30 us), so
//   12544 chunks of four cannot take less than 183 us, whatever the look-back looks like (one level or two, 64 or 256
//   words per trip, four or eight workgroups per CU all gave 179-189 us), and 3136 chunks of sixteen 46 us.
//   With sixteen, a workgroup lives 15 us: ticket 1.8, W 5.5, compaction 2.7, predecessors in the block 2.1, blocks
//   2.1, copy 1.2; a look at another workgroup's word takes 2-4 us while W streams.
//   Variants, each with its best chunk size: chunk = blockIdx instead of a ticket 202 us (workgroups of different
//   XCDs start far out of order and wait for each other); the block's sum kept by atomic adds of every chunk instead
//   of the last chunk's store 258 us (643 us with chunks of four: the adds queue behind the polls of the same
//   address); blocks of 16 or 32 chunks 121 and 114 us; as many persistent workgroups as the device holds, chunks
//   dealt round-robin, the next rows of W requested and the older chunk placed one turn late 241 us (all workgroups
//   then move in lock step with the slowest, two looks per turn behind the loads of W); non-temporal stores and
//   other poll intervals change nothing.
constexpr unsigned kStateSum = 1, kStatePrefix = 2; // 0: nothing published yet
constexpr unsigned kErrSpin = 1, kErrCapacity = 2;
constexpr unsigned kSpinLimit = 1u << 16; // looks at words that are not ready, a few us each
constexpr int      kChunksPerBlock = 64;
constexpr int      kStage = 2048;
constexpr int      kOnePassWaves = 16; // waves = group tiles per chunk: what one ticket buys

struct OnePassHeader {
    unsigned ticket, error, pad0, pad1;
};

__global__ __launch_bounds__(256) void zero_words(unsigned* p, size_t n)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n)
        p[i] = 0;
}

__device__ __forceinline__ unsigned long long word_load(const unsigned long long* p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void word_store(unsigned long long* p, unsigned state, unsigned sum)
{
    __hip_atomic_store(p, ((unsigned long long)state << 32) | sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ unsigned wave_sum(unsigned x)
{
    return (unsigned)__builtin_amdgcn_readlane(wave_inclusive_scan((int)x), 63);
}

// values of the lane's tile whose position p in the group tile's run lies in [lo, lo + kStage) go to out[p - lo];
// kGuard = false: the whole run fits (lo = 0)
template <bool kGuard>
__device__ __forceinline__ void compact_tile(const LaneTile& t, uint16_t* out, int p, int lo)
{
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        const unsigned bits = ((r < 4 ? t.lo : t.hi) >> (8 * (r & 3))) & 0xffu;
        const unsigned d[4] = {t.row[r].x, t.row[r].y, t.row[r].z, t.row[r].w};
#pragma unroll
        for (int c = 0; c < 8; ++c)
            if (bits & (1u << c)) {
                if (!kGuard || (unsigned)(p - lo) < (unsigned)kStage)
                    out[p - lo] = (uint16_t)(d[c >> 1] >> (16 * (c & 1)));
                ++p;
            }
    }
}

__device__ __forceinline__ void wave_lds_fence()
{
    // the wave's own LDS writes are ordered before its reads that follow (lock step: no instruction; the fences hold
    // the compiler to that order although the accesses alias through casts)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__global__ __launch_bounds__(64 * kOnePassWaves, 8) void encode_onepass(
    const uint16_t* __restrict__ W, int K, int G, uint64_t* __restrict__ bitmaps, int* __restrict__ offsets,
    uint16_t* __restrict__ values, unsigned long long capacity, OnePassHeader* __restrict__ head,
    unsigned long long* __restrict__ status, unsigned long long* __restrict__ bword)
{
    __shared__ __attribute__((aligned(16))) uint16_t stage[kOnePassWaves][kStage];
    __shared__ unsigned s_vid, s_excl;
    __shared__ int      s_count[kOnePassWaves];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (threadIdx.x == 0)
        s_vid = __hip_atomic_fetch_add(&head->ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    const unsigned vid    = s_vid; // position of this workgroup in start order = its chunk
    const long     g      = (long)vid * kOnePassWaves + wave;
    const bool     active = g < G;
    int            total = 0, padded = 0, first = 0;
    uint16_t*      out = stage[wave];
    LaneTile       t;
    if (active) {
        t = load_lane_tile(W, K, (int)g, lane);
        bitmaps[(size_t)g * 64 + lane] = ((uint64_t)t.hi << 32) | t.lo;
        const int pc  = __builtin_popcount(t.lo) + __builtin_popcount(t.hi);
        const int inc = wave_inclusive_scan(pc);
        total  = __builtin_amdgcn_readlane(inc, 63);
        first  = inc - pc;
        padded = (total + 7) & ~7;
    }
    if (lane == 0)
        s_count[wave] = padded;
    __syncthreads();
    unsigned agg = 0, before = 0;
#pragma unroll
    for (int w = 0; w < kOnePassWaves; ++w) {
        agg += (unsigned)s_count[w];
        before += w < wave ? (unsigned)s_count[w] : 0u;
    }
    // wave 0 publishes the chunk's sum and requests its first words; they travel while every wave compacts
    const unsigned           blk = vid / kChunksPerBlock, r = vid % kChunksPerBlock;
    const bool               in_block = wave == 0 && (unsigned)lane < r;
    const unsigned long long prefix0  = (unsigned long long)kStatePrefix << 32; // in front of block 0: zero
    long                     idx      = (long)blk - 1 - lane;
    unsigned long long       sa = 0, bp = prefix0;
    if (wave == 0) {
        if (lane == 0)
            word_store(status + vid, kStateSum, agg);
        if (in_block)
            sa = word_load(status + ((long)vid - 1 - lane));
        if (idx >= 0)
            bp = word_load(bword + idx);
    }
    if (active) {
        if (total <= kStage)
            compact_tile<false>(t, out, first, 0);
        else
            compact_tile<true>(t, out, first, 0);
        if (total < kStage && lane < padded - total)
            out[total + lane] = 0;
    }
    if (wave == 0) {
        unsigned spins = 0;
        bool     ok = true;
        while (__ballot(in_block && (unsigned)(sa >> 32) == 0)) { // a predecessor in the block has not published
            if (++spins > kSpinLimit) {
                ok = false;
                break;
            }
            __builtin_amdgcn_s_sleep(4);
            if (in_block)
                sa = word_load(status + ((long)vid - 1 - lane));
        }
        unsigned   excl   = wave_sum(in_block ? (unsigned)sa : 0u);
        const bool closes = r == kChunksPerBlock - 1; // the last chunk of a block speaks for the block
        if (closes && ok && lane == 0)
            word_store(bword + blk, blk == 0 ? kStatePrefix : kStateSum, excl + agg);
        for (long j = (long)blk - 1; ok && j >= 0; j -= 64) {
            int first_pref;
            for (;;) {
                const unsigned long long pref = __ballot((unsigned)(bp >> 32) == kStatePrefix);
                const unsigned long long none = __ballot((unsigned)(bp >> 32) == 0);
                first_pref = pref ? __builtin_ctzll(pref) : 64;
                if ((none ? __builtin_ctzll(none) : 64) >= first_pref)
                    break; // every block this side of the nearest prefix shows its sum
                if (++spins > kSpinLimit) {
                    ok = false;
                    break;
                }
                __builtin_amdgcn_s_sleep(4);
                if (idx >= 0)
                    bp = word_load(bword + idx);
            }
            if (!ok)
                break;
            excl += wave_sum(lane <= first_pref ? (unsigned)bp : 0u);
            if (first_pref < 64)
                break;
            idx -= 64;
            bp = idx >= 0 ? word_load(bword + idx) : prefix0;
        }
        if (lane == 0) {
            if (!ok)
                __hip_atomic_fetch_or(&head->error, kErrSpin, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            else if (closes && blk > 0)
                word_store(bword + blk, kStatePrefix, excl + agg);
            s_excl = excl;
        }
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
    const int n0 = padded < kStage ? padded : kStage;
    for (int i = lane; i < (n0 >> 3); i += 64)
        reinterpret_cast<uint4*>(values + base)[i] = reinterpret_cast<const uint4*>(out)[i];
    if (total > kStage) { // the second half of a group tile more than half full
        wave_lds_fence();
        compact_tile<true>(t, out, first, kStage);
        if (lane < padded - total)
            out[total - kStage + lane] = 0;
        wave_lds_fence();
        for (int i = lane; i < ((padded - kStage) >> 3); i += 64)
            reinterpret_cast<uint4*>(values + base + kStage)[i] = reinterpret_cast<const uint4*>(out)[i];
    }
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
    const size_t G      = (size_t)(M / 64) * (size_t)(K / 64);
    const size_t chunks = (G + spmm_enc::kOnePassWaves - 1) / spmm_enc::kOnePassWaves;
    const size_t blocks = (chunks + spmm_enc::kChunksPerBlock - 1) / spmm_enc::kChunksPerBlock;
    return sizeof(spmm_enc::OnePassHeader) + 8 * (chunks + blocks);
}

extern "C" int SpMM_EncodeDevice_OnePass(hipStream_t stream, const void* W, int M, int K, uint64_t* bitmaps,
                                         int* offsets, void* values, size_t values_capacity, void* scratch)
{
    if (int e = spmm_enc::check(M, K))
        return e;
    if (scratch == nullptr || (reinterpret_cast<uintptr_t>(scratch) & 7) != 0)
        return (int)hipErrorInvalidValue;
    const int    G      = (M / 64) * (K / 64);
    const size_t chunks = ((size_t)G + spmm_enc::kOnePassWaves - 1) / spmm_enc::kOnePassWaves;
    const size_t words  = SpMM_EncodeDevice_ScratchBytes(M, K) / 4;
    (void)hipGetLastError();
    hipLaunchKernelGGL(spmm_enc::zero_words, dim3((unsigned)((words + 255) / 256), 1, 1), dim3(256, 1, 1), 0, stream,
                       static_cast<unsigned*>(scratch), words);
    auto* head   = static_cast<spmm_enc::OnePassHeader*>(scratch);
    auto* status = reinterpret_cast<unsigned long long*>(head + 1);
    hipLaunchKernelGGL(spmm_enc::encode_onepass, dim3((unsigned)chunks, 1, 1), dim3(64 * spmm_enc::kOnePassWaves, 1, 1),
                       0, stream, static_cast<const uint16_t*>(W), K, G, bitmaps, offsets,
                       static_cast<uint16_t*>(values), (unsigned long long)values_capacity, head, status,
                       status + chunks);
    return (int)hipGetLastError();
}
