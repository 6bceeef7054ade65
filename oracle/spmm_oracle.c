/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of the reference's TCA-BME
 * bitmap SpMM path, used as the checker by tests/, by the smoke test and by
 * the benchmark's cpu_baseline leg.  Nothing in the shipped library or its
 * Python host layer links, loads or calls this file.
 *
 * Every function names the reference lines it restates (paths relative to the
 * reference tree).  fp16 is carried as raw uint16_t bit patterns; the two
 * conversion helpers implement IEEE-754 binary16 <-> binary32 with
 * round-to-nearest-even, which is what __half2float / __float2half_rn do.
 *
 * Pinning status
 *   oracle_encode_bitmap   pinned: reference-recorded known answers
 *                          (csrc/out:4,16,28,...), golden vectors written by
 *                          the reference's own encoder compiled from its
 *                          source (oracle/_ref), closed forms (all-zero,
 *                          all-dense, tile index formula), decode(encode)=id.
 *   oracle_decode_bitmap   pinned: inverse of the above on every fixture.
 *   oracle_spmm            pinned against mathematics only: the reference has
 *                          no host SpMM (its checker is cuBLAS on an NVIDIA
 *                          GPU), so this is checked against float64 GEMM
 *                          (numpy) and brute force on tiny shapes.  Parity
 *                          with the reference kernel's own output bits is
 *                          unpinned; the contract is the tolerance
 *                          max|d| <= 1e-2*max|C|, rel-L2 <= 1e-3.
 *   oracle_spmm_bias_act   the same product with bias and activation applied in
 *                          fp32 before the rounding; pinned against float64
 *                          numpy (relu / tanh-form gelu of GEMM + bias) and the
 *                          functions' closed-form properties.
 *   oracle_splitk_*        pinned: partition closed form + sum over batches
 *                          equals the unsplit product.
 *   oracle_init_host_matrices  pinned: reproduces the seven recorded
 *                          (M, G, NNZ, max_nnz) tuples bit-for-bit.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ fp16 */

float oracle_half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp  = (h >> 10) & 0x1fu;
    uint32_t man  = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: renormalise */
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while ((man & 0x400u) == 0);
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t oracle_float_to_half(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) { /* inf / nan */
        if (absx > 0x7f800000u)
            return (uint16_t)(sign | 0x7e00u | ((absx >> 13) & 0x3ffu));
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absx >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absx < 0x33000001u) { /* below half of the smallest subnormal */
        return sign;
    }
    int32_t  e = (int32_t)(absx >> 23) - 127;
    uint32_t m = (absx & 0x7fffffu) | 0x800000u;
    int      shift;
    uint32_t base;
    if (e < -14) { /* subnormal result */
        shift = 13 + (-14 - e);
        base  = 0;
    } else {
        shift = 13;
        base  = (uint32_t)(e + 15) << 10;
        m &= 0x7fffffu;
    }
    uint32_t q    = m >> shift;
    uint32_t rem  = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u)))
        q++;
    return (uint16_t)(sign | (base + q)); /* carry into exponent is correct */
}

/* --------------------------------------------------------------- encoder */

/*
 * csrc/SpMM_API.cuh:112-241 (InitSparseMatrixA_bitmap), called with
 * tile_M=8, tile_M_median=16, tile_M_global=64, tile_K=8, tile_K_median=64,
 * tile_K_global=64 at every reference call site (csrc/SpMM_API.cuh:275,
 * kernel_benchmark/spmm_test.cu:316).  The loop nest below keeps the
 * reference's traversal order, which is what fixes the memory format:
 *   64x64 group tiles row-major (:153-154); inside one, four 16-row strips
 *   (:162); inside a strip, column pairs of 8x8 tiles left to right (:168)
 *   and, per pair, the 2x2 quad in column-major order (:170-171); inside an
 *   8x8 tile a row-major scan sets bit r*8+c (:182-190).
 * A value is kept iff its float value != 0.0f (:189): -0.0 is dropped, NaN
 * and subnormals are kept.  Each group tile's values are padded with +0.0 to
 * a multiple of 8 (:216-220).  tile_cnt is the per-8x8 count the reference
 * names TileOffsets (:201); median holds the four strip start offsets inside
 * each group tile (:160,:207-211); global is the exclusive prefix sum of the
 * padded counts (:231-235); *max_nnz is the largest padded count (:224-226).
 * Returns the number of group tiles, or -1 if an allocation fails (:141-144).
 * Buffers are malloc'd and owned by the caller, like the reference's.
 */
int oracle_encode_bitmap(const uint16_t* A, int M, int K, uint16_t** vals_out, int** tile_cnt_out,
                         int** median_out, int** global_out, uint64_t** bitmap_out, int* max_nnz)
{
    const int gm_n = M / 64, gk_n = K / 64;
    const int G    = gm_n * gk_n;
    const int T    = (M / 8) * (K / 8);

    uint16_t* vals     = (uint16_t*)malloc((size_t)M * K * sizeof(uint16_t) + 16);
    int*      tile_cnt = (int*)malloc((size_t)(T > 0 ? T : 1) * sizeof(int));
    int*      median   = (int*)malloc((size_t)(G > 0 ? G : 1) * 4 * sizeof(int));
    int*      global   = (int*)malloc((size_t)(G + 1) * sizeof(int));
    uint64_t* bitmap   = (uint64_t*)malloc((size_t)(T > 0 ? T : 1) * sizeof(uint64_t));
    if (!vals || !tile_cnt || !median || !global || !bitmap) {
        free(vals), free(tile_cnt), free(median), free(global), free(bitmap);
        return -1;
    }

    int n = 0, t = 0, mi = 0;
    *max_nnz  = 0;
    global[0] = 0;
    for (int gm = 0; gm < gm_n; ++gm) {
        for (int gk = 0; gk < gk_n; ++gk) {
            int in_group = 0;
            median[mi++] = 0;
            for (int strip = 0; strip < 4; ++strip) {
                for (int kpair = 0; kpair < 8; kpair += 2) {
                    for (int j = 0; j < 2; ++j) {
                        for (int i = 0; i < 2; ++i) {
                            const int row0 = gm * 64 + strip * 16 + i * 8;
                            const int col0 = gk * 64 + (kpair + j) * 8;
                            uint64_t  bm   = 0;
                            int       cnt  = 0;
                            for (int r = 0; r < 8; ++r) {
                                for (int c = 0; c < 8; ++c) {
                                    uint16_t v = A[(size_t)(row0 + r) * K + col0 + c];
                                    if (oracle_half_to_float(v) != 0.0f) {
                                        bm |= 1ULL << (r * 8 + c);
                                        vals[n++] = v;
                                        cnt++;
                                    }
                                }
                            }
                            bitmap[t]   = bm;
                            tile_cnt[t] = cnt;
                            t++;
                            in_group += cnt;
                        }
                    }
                }
                if (strip < 3)
                    median[mi++] = in_group;
            }
            int pad = (8 - in_group % 8) % 8;
            for (int p = 0; p < pad; ++p)
                vals[n++] = 0;
            in_group += pad;
            global[gm * gk_n + gk + 1] = global[gm * gk_n + gk] + in_group;
            if (in_group > *max_nnz)
                *max_nnz = in_group;
        }
    }
    uint16_t* shrunk = (uint16_t*)realloc(vals, (size_t)(n > 0 ? n : 1) * sizeof(uint16_t));
    *vals_out        = shrunk ? shrunk : vals;
    *tile_cnt_out    = tile_cnt;
    *median_out      = median;
    *global_out      = global;
    *bitmap_out      = bitmap;
    return G;
}

/* Caller-side rounding of max_nnz to a multiple of 64
 * (csrc/SpMM_API.cuh:284-286, kernel_benchmark/spmm_test.cu:325-327). */
int oracle_round_max_nnz(int max_nnz)
{
    return (max_nnz % 64 != 0) ? ((max_nnz / 64) + 1) * 64 : max_nnz;
}

void oracle_free(void* p)
{
    free(p);
}

/* --------------------------------------------------------------- decoder */

/*
 * Inverse of the encoder, following how the kernel addresses the format:
 * group tile g = y*(K/64)+k starts at values[global[g]] and owns bitmaps
 * [64g, 64g+64) (csrc/SpMM_Kernel.cuh:44-46,82-84); bitmaps are consumed in
 * storage order, each bit taking the next compact value
 * (csrc/MatMulUtilities.cuh:27-57).  Storage index -> coordinates:
 *   t = 64g + 16*strip + 4*q + 2*j + i  covers rows 64gm+16strip+8i..+7,
 *   columns 64gk+16q+8j..+7; bit r*8+c is element (r, c) of that tile.
 * W must hold M*K entries; it is fully overwritten (zeros are +0.0).
 */
void oracle_decode_bitmap(const uint16_t* vals, const uint64_t* bitmap, const int* global, int M, int K,
                          uint16_t* W)
{
    const int gk_n = K / 64;
    memset(W, 0, (size_t)M * K * sizeof(uint16_t));
    for (int gm = 0; gm < M / 64; ++gm) {
        for (int gk = 0; gk < gk_n; ++gk) {
            const int g = gm * gk_n + gk;
            int       p = global[g];
            for (int lt = 0; lt < 64; ++lt) {
                const int strip = lt >> 4, q = (lt >> 2) & 3, j = (lt >> 1) & 1, i = lt & 1;
                const int row0 = gm * 64 + strip * 16 + i * 8;
                const int col0 = gk * 64 + q * 16 + j * 8;
                uint64_t  bm   = bitmap[(size_t)g * 64 + lt];
                for (int b = 0; b < 64; ++b)
                    if ((bm >> b) & 1ULL)
                        W[(size_t)(row0 + (b >> 3)) * K + col0 + (b & 7)] = vals[p++];
            }
        }
    }
}

/* ------------------------------------------------------------------ SpMM */

/*
 * Split-K partition of the K/64 group-tile columns
 * (csrc/SpMM_Kernel.cuh:35-43): every batch gets avg = ceil(nkb/split_k)
 * columns starting at batch*avg and the last batch what remains
 * (avg - (avg*split_k - nkb)).  For split_k values where that remainder
 * formula leaves an earlier batch reaching past the matrix (e.g. nkb=5,
 * split_k=4) the reference kernel would walk into the next row block; here a
 * batch is clamped to the columns that exist, which is the same partition
 * whenever the reference's is in bounds.  Returns the first column and
 * writes the count.
 */
int oracle_splitk_range(int K, int split_k, int batch, int* count)
{
    const int nkb   = K / 64;
    const int avg   = (nkb - 1) / split_k + 1;
    const int first = batch * avg;
    int       cnt   = nkb - first;
    if (cnt > avg)
        cnt = avg;
    if (cnt < 0)
        cnt = 0;
    *count = cnt;
    return first;
}

/*
 * Host statement of what SpMM_SplitK_API_bitmap_v3 computes
 * (csrc/SpMM_API.cuh:47-110): C[m + n*M] = fp16( sum_k fp32(W[m][k]) *
 * fp32(X[k + n*K]) ), W taken from the compressed arrays, X and C in the
 * reference's layouts (kernel_benchmark/spmm_test.cu:38-39: X is [N][K],
 * C is [N][M]), fp32 accumulation (csrc/MMA_PTX.cuh:120-139), fp16
 * round-to-nearest store (csrc/SpMM_Kernel.cuh:198).
 *
 * split_k == 1: one fp32 sum over the whole K range.
 * split_k  > 1: one partial per batch of oracle_splitk_range.  With
 *   partial_fp16 != 0 each partial is rounded to fp16 before the final fp32
 *   sum, as the reference's slabs are (csrc/SpMM_Kernel.cuh:192-198,
 *   csrc/Reduction_Kernel.cuh:36-44); with partial_fp16 == 0 the partials
 *   stay fp32.
 * The accumulation order inside a batch is ascending k (the kernel's order is
 * an implementation detail; the tolerance in the tests absorbs it).
 */
/* act: 0 none, 1 ReLU, 2 GELU (tanh form, as FasterTransformer's gelu) */
static float oracle_activation(float x, int act)
{
    if (act == 1)
        return x > 0.f ? x : (x == x ? 0.f : x);
    if (act == 2)
        return 0.5f * x * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
    return x;
}

/* SpMM with the element-wise tail of the reference's FfnLayer folded in before the fp16 rounding
 * (third_party/ft_spinfer.patch:766-768): C = fp16(act(sum + bias[m])).  bias may be NULL. */
void oracle_spmm_bias_act(const uint16_t* vals, const uint64_t* bitmap, const int* global, const uint16_t* X,
                          uint16_t* C, int M, int N, int K, int split_k, int partial_fp16, const uint16_t* bias,
                          int act)
{
    if (split_k < 1)
        split_k = 1;
    const int gk_n = K / 64;
#pragma omp parallel
    {
        float* wrow = (float*)malloc(64 * 64 * sizeof(float));
        float* xt   = (float*)malloc((size_t)64 * N * sizeof(float));
        float* acc  = (float*)malloc((size_t)64 * N * sizeof(float));
        float* tot  = (float*)malloc((size_t)64 * N * sizeof(float));
#pragma omp for schedule(dynamic, 1)
        for (int gm = 0; gm < M / 64; ++gm) {
            for (int e = 0; e < 64 * N; ++e)
                tot[e] = 0.f;
            for (int b = 0; b < split_k; ++b) {
                int cnt, first = oracle_splitk_range(K, split_k, b, &cnt);
                for (int e = 0; e < 64 * N; ++e)
                    acc[e] = 0.f;
                for (int gk = first; gk < first + cnt; ++gk) {
                    const int g = gm * gk_n + gk;
                    int       p = global[g];
                    memset(wrow, 0, 64 * 64 * sizeof(float));
                    for (int lt = 0; lt < 64; ++lt) {
                        const int strip = lt >> 4, q = (lt >> 2) & 3, j = (lt >> 1) & 1, i = lt & 1;
                        const int r0 = strip * 16 + i * 8, c0 = q * 16 + j * 8;
                        uint64_t  bm = bitmap[(size_t)g * 64 + lt];
                        for (int bit = 0; bit < 64; ++bit)
                            if ((bm >> bit) & 1ULL)
                                wrow[(r0 + (bit >> 3)) * 64 + c0 + (bit & 7)] = oracle_half_to_float(vals[p++]);
                    }
                    for (int n = 0; n < N; ++n)
                        for (int k = 0; k < 64; ++k)
                            xt[n * 64 + k] = oracle_half_to_float(X[(size_t)n * K + gk * 64 + k]);
                    for (int r = 0; r < 64; ++r)
                        for (int n = 0; n < N; ++n) {
                            float s = acc[n * 64 + r];
                            for (int k = 0; k < 64; ++k)
                                s += wrow[r * 64 + k] * xt[n * 64 + k];
                            acc[n * 64 + r] = s;
                        }
                }
                for (int e = 0; e < 64 * N; ++e) {
                    float v = acc[e];
                    if (split_k > 1 && partial_fp16)
                        v = oracle_half_to_float(oracle_float_to_half(v));
                    tot[e] += v;
                }
            }
            for (int n = 0; n < N; ++n)
                for (int r = 0; r < 64; ++r)
                {
                    float v = tot[n * 64 + r];
                    if (bias)
                        v += oracle_half_to_float(bias[gm * 64 + r]);
                    C[(size_t)n * M + gm * 64 + r] = oracle_float_to_half(oracle_activation(v, act));
                }
        }
        free(wrow), free(xt), free(acc), free(tot);
    }
}

void oracle_spmm(const uint16_t* vals, const uint64_t* bitmap, const int* global, const uint16_t* X,
                 uint16_t* C, int M, int N, int K, int split_k, int partial_fp16)
{
    oracle_spmm_bias_act(vals, bitmap, global, X, C, M, N, K, split_k, partial_fp16, NULL, 0);
}

int oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* Dense float64 product of fp16 operands, same layouts; for cross-checks. */
void oracle_gemm_f64(const uint16_t* W, const uint16_t* X, double* C, int M, int N, int K)
{
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            double s = 0.0;
            for (int k = 0; k < K; ++k)
                s += (double)oracle_half_to_float(W[(size_t)m * K + k]) *
                     (double)oracle_half_to_float(X[(size_t)n * K + k]);
            C[(size_t)n * M + m] = s;
        }
}

/* ----------------------------------------------------- reference harness */

/*
 * kernel_benchmark/spmm_test_utils.h:88-102 (init_host_matrices): glibc
 * rand(), two draws per kept weight, one per activation.  The reference never
 * seeds it; pass reseed=1 to call srand(1), which is the state an unseeded
 * process starts in.
 */
void oracle_init_host_matrices(uint16_t* a, uint16_t* b, int M, int K, int N, int pruning_percentage, int reseed)
{
    if (reseed)
        srand(1);
    for (int i = 0; i < M; i++)
        for (int j = 0; j < K; j++) {
            int r = rand() % 100;
            if (r >= pruning_percentage)
                a[j + (size_t)i * K] = oracle_float_to_half((float)(rand() % 5) / 5 - 0.5f);
            else
                a[j + (size_t)i * K] = oracle_float_to_half(0.0f);
        }
    for (size_t i = 0; i < (size_t)N * K; i++)
        b[i] = oracle_float_to_half((float)(rand() % 5) / 5 - 0.5f);
}

/* kernel_benchmark/spmm_test_utils.h:104-110 (ComputeTotalError). */
double oracle_total_error(const uint16_t* ref, const uint16_t* other, int m, int n)
{
    double e = 0.0;
    for (size_t i = 0; i < (size_t)m * n; i++)
        e += fabs((double)oracle_half_to_float(ref[i]) - (double)oracle_half_to_float(other[i]));
    return e;
}

/* csrc/Reduction_Kernel.cuh:24-45: C[i] = fp16( sum_s fp32(ws[s*M*N + i]) ). */
void oracle_splitk_reduce_fp16(const uint16_t* ws, uint16_t* C, int M, int N, int split_k)
{
    const size_t mn = (size_t)M * N;
    for (size_t i = 0; i < mn; ++i) {
        float s = 0.f;
        for (int b = 0; b < split_k; ++b)
            s += oracle_half_to_float(ws[(size_t)b * mn + i]);
        C[i] = oracle_float_to_half(s);
    }
}
