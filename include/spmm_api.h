/*
 * C ABI of libSpMM_API.so for gfx950 (MI355X): bitmap-compressed (TCA-BME)
 * unstructured-sparse SpMM,  C[M x N] = W[M x K] (sparse fp16) * X[K x N]
 * (dense fp16), fp32 accumulation, fp16 output.
 *
 * The library keeps the surface of the reference's libSpMM_API.so: a host
 * encoder and a split-K SpMM entry point.  Each declaration cites the
 * reference interface it replaces (paths relative to the reference tree).
 *
 * Data layouts (identical to the reference's, so encoded weights and
 * activations are interchangeable):
 *   W        row-major [M][K] fp16 on the host (encoder input only).
 *   values   compact non-zero fp16 values, group tile after group tile; each
 *            64x64 group tile's run is zero-padded to a multiple of 8 halves,
 *            so every run starts 16-byte aligned.
 *   bitmaps  one uint64 per 8x8 tile, 64 per group tile; bit r*8+c is element
 *            (r, c).  Storage index of a tile:
 *            t = 64*g + 16*strip + 4*q + 2*j + i,  g = gm*(K/64) + gk,
 *            rows 64*gm + 16*strip + 8*i .. +7, columns 64*gk + 16*q + 8*j .. +7.
 *   offsets  (TileOffsets_global) G+1 ints, exclusive prefix sum of the padded
 *            per-group-tile value counts; G = (M/64)*(K/64).
 *   X        [N][K] fp16 (element (k, n) at X[k + n*K]).
 *   C        [N][M] fp16 (element (m, n) at C[m + n*M]); fully overwritten.
 * M and K must be multiples of 64.  N must be 8, 16, 32, 64 or a multiple
 * of 128.  All SpMM pointer arguments are device memory; calls are
 * asynchronous on `stream` and never synchronise the host.
 *
 * fp16 buffers are typed `void*` / `uint16_t*` so that this header needs no
 * HIP header; `half*` arguments convert implicitly.
 */
#ifndef SPMM_API_H
#define SPMM_API_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef HIP_INCLUDE_HIP_HIP_RUNTIME_API_H
typedef struct ihipStream_t* hipStream_t;
typedef struct ihipEvent_t*  hipEvent_t;
#endif

/*
 * SpMM, north-star form.  Replaces SpMM_SplitK_API_bitmap_v3
 * (csrc/SpMM_API.cuh:47-110; original 14-argument dense-X form as called at
 * kernel_benchmark/spmm_test.cu:375-388 and third_party/ft_spinfer.patch:3736-3749)
 * with the arguments the gfx950 kernel actually needs: strip offsets and the
 * max-nnz hint are derived from the bitmaps on the device.
 *
 *   Split_K >= 1  use that many K batches (partition as in
 *                 csrc/SpMM_Kernel.cuh:35-43);
 *   Split_K <= 0  the library picks one for the shape (SpMM_SplitK_Auto).
 * `workspace` must hold SpMM_WorkspaceBytes(M, N, K, Split_K) bytes (call it
 * with the same Split_K argument, <= 0 included): partial sums are kept in
 * fp32 (4*M*N*Split_K bytes for an explicit Split_K > 1) and reduced to fp16
 * by a second kernel.  It may be NULL when that size is 0.  Its contents on
 * entry do not matter.
 * Returns a hipError_t value as int: 0 on success; 999 (hipErrorUnknown) with
 * the reference's message for an unsupported N (csrc/SpMM_API.cuh:91-94);
 * 1 (hipErrorInvalidValue) for M or K not a multiple of 64, a missing
 * workspace, or a pointer that is NULL or not aligned as the kernels need
 * (values, X, C and workspace 16 bytes, bitmaps 8, offsets 4: refused on the
 * host, where the reference would fault on the device); otherwise the launch
 * status (csrc/SpMM_API.cuh:99-109).  The same holds for the other SpMM
 * entry points below.
 */
int SpMM_SplitK_API(hipStream_t stream, const void* values, const uint64_t* bitmaps, const int* offsets,
                    const void* X, void* C, int M, int N, int K, void* workspace, int Split_K);

/*
 * SpMM_SplitK_API with the size of `workspace` stated: the same call, except that it returns 1
 * (hipErrorInvalidValue) without launching anything when the split the call resolves to needs more than
 * `workspace_bytes`.  For callers that pass Split_K <= 0: between their SpMM_WorkspaceBytes(.., 0) and the call,
 * the library's choice for the shape may have changed (SpMM_SplitK_TableSet/TableLoad, SPMM_SPLITK_TABLE read at
 * first use), and SpMM_SplitK_API has no way to notice that the buffer is now too small.  The reference's call
 * (csrc/SpMM_API.cuh:47-110) takes Split_K from its caller only and has no such case.
 */
int SpMM_SplitK_API_Sized(hipStream_t stream, const void* values, const uint64_t* bitmaps, const int* offsets,
                          const void* X, void* C, int M, int N, int K, void* workspace, size_t workspace_bytes,
                          int Split_K);

/*
 * SpMM, reference call-site form: same argument order as the 14-argument
 * SpMM_SplitK_API_bitmap_v3 the reference's callers use
 * (kernel_benchmark/spmm_test.cu:375-388, third_party/ft_spinfer.patch:3736-3749),
 * with hipStream_t for cudaStream_t, so those callers port by type
 * substitution.  `A` (dense W) is unused and may be NULL, as in the reference.
 * `TileOffsets` is TileOffsets_global.  `TileOffsets_Median` and
 * `max_nnz_intile` are accepted for compatibility and not read.
 * The workspace contract is the reference's: M*N*Split_K halves
 * (kernel_benchmark/spmm_test.cu:361), partial sums stored as fp16
 * (csrc/SpMM_Kernel.cuh:192-198) and summed in fp32
 * (csrc/Reduction_Kernel.cuh:24-45).  Split_K must be >= 1.
 */
int SpMM_SplitK_API_bitmap_v3(hipStream_t stream, const void* A, const void* Compressed_A, const int* TileOffsets,
                              const int* TileOffsets_Median, const uint64_t* bitmap, const int* max_nnz_intile,
                              const void* B, void* C, int M_Global, int N_Global, int K_Global,
                              void* Reduction_Workspace, int Split_K);

/*
 * Split_K the library would pick for a shape when asked to (Split_K <= 0).
 * Replaces the offline per-matrix table SplitKDict
 * (end2end_inference/ft_tools/huggingface_opt_convert_Phase2.py:23).
 */
int SpMM_SplitK_Auto(int M, int N, int K);
/* The built-in cost model's choice for the shape, whatever the table of measured choices (below) holds. */
int SpMM_SplitK_CostModel(int M, int N, int K);

/*
 * Measured Split_K choices, which SpMM_SplitK_Auto (and every call with Split_K <= 0) prefers to its built-in
 * cost model.  They take the place of the hand-kept tables of the reference: SplitKDict
 * (end2end_inference/ft_tools/huggingface_opt_convert_Phase2.py:23, keyed by M alone) and the SPLIT_K array of
 * kernel_benchmark/run_all_main.sh:5.  The table is keyed by (M, N, K) and shared by all threads of the process.
 *   TableSet    records one choice; returns 0, or hipErrorInvalidValue for a shape the library does not run.
 *   TableSetMany records `count` choices at once, `entries` holding {M, N, K, Split_K} four ints each (one copy of
 *               the table instead of one per entry); returns 0, or hipErrorInvalidValue, recording nothing, when
 *               any entry is one TableSet would refuse.
 *   TableLoad   adds the entries of a text file of "M N K Split_K" lines ('#' starts a comment); returns their
 *               number, -1 if the file cannot be opened, -2 on a malformed line.
 *   TableSave   writes the table in that format; returns the number of entries, -1 if the file cannot be written.
 *   TableClear  empties the table.
 * The first time a choice is needed a file is loaded: the one SPMM_SPLITK_TABLE names in the environment, or, when
 * that variable is not set, the measured table shipped with the library (tuned/splitk_mi355x.txt beside the
 * library's directory) if it is there.  SPMM_SPLITK_TABLE set to an empty string loads nothing (cost model only).
 * A workspace must be sized (SpMM_WorkspaceBytes) after the table is in its final state.
 */
int  SpMM_SplitK_TableSet(int M, int N, int K, int Split_K);
int  SpMM_SplitK_TableSetMany(const int* entries, int count);
int  SpMM_SplitK_TableLoad(const char* path);
int  SpMM_SplitK_TableSave(const char* path);
void SpMM_SplitK_TableClear(void);

/* Bytes of workspace SpMM_SplitK_API needs for this call (0 for Split_K == 1).
 * Split_K <= 0 means the library's own choice and returns a size that covers
 * whatever way it may split the work. */
size_t SpMM_WorkspaceBytes(int M, int N, int K, int Split_K);

/*
 * SpMM with bias and activation folded into the output pass:
 *   C[m + n*M] = fp16( act( sum_k W[m][k] * X[k][n]  +  bias[m] ) ),   everything before the cast in fp32.
 * Takes the place of the SpMM call followed by the element-wise add-bias / activation kernels of the reference's
 * FasterTransformer layer (third_party/ft_spinfer.patch:766-768 and the unpatched FfnLayer code around it); no
 * such entry point exists in the reference's library.  `bias` is M fp16 values on the device, or NULL.
 * `activation`: 0 none, 1 ReLU, 2 GELU in its tanh form 0.5*x*(1 + tanh(0.79788456*(x + 0.044715*x^3))).
 * The partial sums always pass through `workspace` (fp32), which must hold
 * SpMM_WorkspaceBytesBiasAct(M, N, K, Split_K) bytes = 4*M*N*max(Split_K, 1), also for an unsplit K.
 * Other arguments, Split_K <= 0 and return values as for SpMM_SplitK_API; an unknown activation returns 1.
 */
int SpMM_SplitK_API_BiasAct(hipStream_t stream, const void* values, const uint64_t* bitmaps, const int* offsets,
                            const void* X, void* C, int M, int N, int K, void* workspace, int Split_K,
                            const void* bias, int activation);
size_t SpMM_WorkspaceBytesBiasAct(int M, int N, int K, int Split_K);

/*
 * SpMM_SplitK_API without a workspace argument and without any allocation.  It has no counterpart in the
 * reference; it is for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  The fp32 partial sums of a split K go to a device array of
 * SPMM_NOALLOC_SCRATCH_BYTES that the library itself holds on every GPU it runs on until the process ends.
 * Arguments and results are those of SpMM_SplitK_API (the same kernels run).  An explicit Split_K whose partial
 * sums (4*M*N*Split_K bytes for Split_K > 1) exceed the array prints a message and returns 1
 * (hipErrorInvalidValue) without launching anything.  With Split_K <= 0 the library's own choice gives way to the
 * largest split whose partial sums fit (an unsplit K needs none, so such a call always runs);
 * SpMM_SplitK_AutoNoAlloc reports that split.  The call makes no hipMalloc/hipFree; the first call on a
 * device looks up the array's device address once (make that call outside a graph capture).
 * All calls on one GPU share the array: calls that overlap in time on one GPU (different streams, or graphs
 * replayed concurrently) race on it and must be serialised by the caller.
 */
#define SPMM_NOALLOC_SCRATCH_BYTES (32u << 20)
int SpMM_SplitK_API_NoAlloc(hipStream_t stream, const void* values, const uint64_t* bitmaps, const int* offsets,
                            const void* X, void* C, int M, int N, int K, int Split_K);
int SpMM_SplitK_AutoNoAlloc(int M, int N, int K);

/*
 * Host encoder, C twin of InitSparseMatrixA_bitmap
 * (csrc/SpMM_API.cuh:112-241): dense row-major fp16 W -> TCA-BME arrays.
 * Output is bit-identical to the reference's.  The tile-size arguments are
 * kept for signature compatibility and must be 8,16,64,8,64,64 (the only
 * values any reference call site passes); anything else returns -2.
 * The five output buffers are malloc'd and owned by the caller (free()):
 *   Compressed_Val      TileOffsets_global[G] halves
 *   TileOffsets         per-8x8-tile non-zero counts, (M/8)*(K/8) ints
 *   TileOffsets_median  4*G ints, strip start offsets inside each group tile
 *   TileOffsets_global  G+1 ints
 *   bitmap              (M/8)*(K/8) uint64
 * *max_nnz_count receives the largest padded per-group-tile count (callers
 * round it up to a multiple of 64, csrc/SpMM_API.cuh:284-286).
 * Returns G = (M/64)*(K/64), or -1 if an allocation fails (:141-144).
 * Rows/columns beyond the last multiple of 64 are ignored, as in the
 * reference (:130-132).
 */
int InitSparseMatrixA_bitmap(uint16_t* A_h, int M, int K, int tile_M, int tile_M_median, int tile_M_global,
                             int tile_K, int tile_K_median, int tile_K_global, uint16_t** Compressed_Val,
                             int** TileOffsets, int** TileOffsets_median, int** TileOffsets_global,
                             uint64_t** bitmap, int* max_nnz_count);

/*
 * Device encoder: the same arrays as InitSparseMatrixA_bitmap, bit for bit, from a dense row-major fp16 W that
 * already sits in device memory (no counterpart in the reference, whose only encoder is the single-threaded host
 * function csrc/SpMM_API.cuh:112-241).  M and K must be multiples of 64 (else 1, hipErrorInvalidValue).
 * All pointers are device memory; both calls are asynchronous on `stream`.
 *   SpMM_EncodeDevice_Bitmaps  writes `bitmaps` (64*G uint64) and `offsets` (TileOffsets_global, G+1 ints),
 *                              G = (M/64)*(K/64).
 *   (the caller reads offsets[G], the number of halves `values` must hold, and allocates it)
 *   SpMM_EncodeDevice_Values   writes `values` (compact non-zeros, every group tile's run zero-padded to a
 *                              multiple of 8), given the `offsets` of the first call.
 * The per-tile counts, strip offsets and max-nnz hint of the host encoder are not produced: the SpMM entry points
 * of this library do not read them.
 */
int SpMM_EncodeDevice_Bitmaps(hipStream_t stream, const void* W, int M, int K, uint64_t* bitmaps, int* offsets);
int SpMM_EncodeDevice_Values(hipStream_t stream, const void* W, int M, int K, const int* offsets, void* values);

/*
 * The device encoder in one pass over W (the two calls above read W twice): the same three arrays, bit for bit,
 * from one kernel, for a caller that can give `values` room before the number of values is known.  The faster form
 * (about 0.6 of the time of the two calls on a 28672 x 7168 matrix).
 *   values_capacity  halves `values` can hold; M*K always suffices.  offsets[G] is the number actually written.
 *   scratch          SpMM_EncodeDevice_ScratchBytes(M, K) bytes of device memory, 8-byte aligned, contents
 *                    irrelevant on entry (the call clears it).  After the call has finished, scratch's second
 *                    32-bit word is 0 on success; bit 1 (value 2) says `values` was too small (bitmaps and offsets
 *                    are complete, some runs were not written), bit 0 that a workgroup gave up waiting for its
 *                    predecessors (nothing is valid then; not expected on a healthy device).
 * Asynchronous on `stream`; returns the launch status, or 1 for M or K not a multiple of 64 or a missing or
 * misaligned scratch.  No counterpart in the reference.
 */
size_t SpMM_EncodeDevice_ScratchBytes(int M, int K);
int    SpMM_EncodeDevice_OnePass(hipStream_t stream, const void* W, int M, int K, uint64_t* bitmaps, int* offsets,
                                 void* values, size_t values_capacity, void* scratch);

/*
 * File-to-file encoder, replaces Our_GenSparseMatrixBinFile
 * (csrc/SpMM_API.cuh:243-320; called through ctypes at
 * end2end_inference/ft_tools/huggingface_opt_convert_Phase2.py:88-102).
 * Reads M*K fp16 from DenseMatrixFileName and writes the six files the
 * reference writes, byte for byte: values, TileOffsets_global (G+1 ints),
 * TileOffsets_median (4G ints), bitmaps (64G uint64), max_nnz rounded up to a
 * multiple of 64 (1 int), and sizes {val_count, G+1, 4G, 64G} (4 ints).
 * Like the reference it prints a message and exits the process with -1 when a
 * file cannot be opened or is too short.
 */
void Our_GenSparseMatrixBinFile(char* DenseMatrixFileName, int M, int K, char* Compressed_ValFileName,
                                char* bitmap_TileOffsets_globalFileName, char* bitmap_TileOffsets_medianFileName,
                                char* bitmapFileName, char* max_nnz_intileFileName, char* OutputSizesFileName);

/*
 * Readers of the six files Our_GenSparseMatrixBinFile writes: the consumer side, which in the reference is the
 * FasterTransformer layer-weight loader (third_party/ft_spinfer.patch:2335-2357: loadDataArrayFromBin of
 * .NZWeights/.gtile/.mtile/.ltile/.intile into device arrays sized from the model's configuration).
 *   SpMM_ReadWeightFiles  reads them into malloc'd host arrays (free() each): values (val_count halves),
 *                         TileOffsets_global (G+1 ints), TileOffsets_median (4G ints), bitmap (64G uint64) and the
 *                         max-nnz hint.  TileOffsets_median, max_nnz_intile and val_count may be NULL.
 *   SpMM_LoadWeightFiles  reads them and leaves them in device memory of the current device (hipMalloc +
 *                         synchronous copies), ready to be passed to the SpMM entry points; median_d, max_nnz_d
 *                         and val_count may be NULL (then those are not kept).  Release with SpMM_FreeWeights.
 * Both check the sizes file against M and K ({val_count, G+1, 4G, 64G}, csrc/SpMM_API.cuh:304-308), every file's
 * length and that the offsets start at 0, end at val_count and grow by multiples of 8 of at most 4096.
 * Return G = (M/64)*(K/64), or -1 a file is missing or has another length, -2 the files do not match M and K or
 * each other, -4 a required argument is NULL, -5 (Load only) a HIP call failed; nothing is returned or kept then.
 * Unlike the reference's loader they never end the process.
 */
int  SpMM_ReadWeightFiles(const char* Compressed_ValFileName, const char* TileOffsets_globalFileName,
                          const char* TileOffsets_medianFileName, const char* bitmapFileName,
                          const char* max_nnz_intileFileName, const char* OutputSizesFileName, int M, int K,
                          uint16_t** Compressed_Val, int** TileOffsets_global, int** TileOffsets_median,
                          uint64_t** bitmap, int* max_nnz_intile, int* val_count);
int  SpMM_LoadWeightFiles(const char* Compressed_ValFileName, const char* TileOffsets_globalFileName,
                          const char* TileOffsets_medianFileName, const char* bitmapFileName,
                          const char* max_nnz_intileFileName, const char* OutputSizesFileName, int M, int K,
                          void** values_d, int** offsets_d, int** median_d, uint64_t** bitmaps_d, int** max_nnz_d,
                          int* val_count);
void SpMM_FreeWeights(void* values_d, int* offsets_d, int* median_d, uint64_t* bitmaps_d, int* max_nnz_d);

/*
 * Timing aid with no counterpart in the reference (its harness times whole
 * calls with cudaEvents, kernel_benchmark/spmm_test.cu:374-411): the next SpMM
 * call made by this thread attaches the two events to the dispatch of its main
 * kernel, so that `before_main` carries the kernel's begin timestamp and
 * `after_main` its end timestamp; hipEventElapsedTime between them is the main
 * kernel's duration alone (no launch latency, no split-K reduction).  Either
 * may be NULL.  The request is consumed by that one call.
 */
void SpMM_TimeNextCall(hipEvent_t before_main, hipEvent_t after_main);

/*
 * Reporting aid with no counterpart in the reference: launches one wave on `stream` that idles for about `spin_us`
 * microseconds (1..100000) and writes two 64-bit counts to `ticks_d` (device memory, 16 bytes): by how much the
 * shader-clock counter and the constant 100 MHz counter advanced meanwhile.  100 * ticks_d[0] / ticks_d[1] is the
 * shader clock in MHz during that time; run on a second stream beside SpMM calls it is the clock those calls run
 * at, which lets timings taken on different machines be compared in cycles.  Returns the launch status.
 */
int SpMM_ShaderClockProbe(hipStream_t stream, unsigned long long* ticks_d, int spin_us);

/*
 * Name of the main kernel a call of SpMM_SplitK_API, SpMM_SplitK_API_Sized or SpMM_SplitK_API_NoAlloc with these
 * dimensions dispatches, as a profiler prints it, e.g. "spmm::spmm_bitmap_rows<1, true>" (second template argument:
 * fp32 partial sums to the workspace, which these three entry points use whenever K is split).  It does not hold
 * for SpMM_SplitK_API_bitmap_v3 (fp16 partial sums: "false" for every split) or SpMM_SplitK_API_BiasAct (one fp32
 * slab even for an unsplit K: "true" for every split).  Split_K <= 0 asks for the library's own split.  Reporting aid for benchmarks that key profiler records by kernel; no
 * reference counterpart.  The string belongs to the library and is valid until the thread's next call of this
 * function; NULL for dimensions the SpMM calls refuse.
 */
const char* SpMM_KernelName(int M, int N, int K, int Split_K);

/* Library version string, e.g. "spmm-gfx950 0.1". */
const char* SpMM_Version(void);

#ifdef __cplusplus
} /* extern "C" */

#if defined(HIP_INCLUDE_HIP_HIP_FP16_H) || defined(SPMM_API_WITH_HALF)
/*
 * C++ overload with the reference's exact signature and mangled name
 * (_Z24InitSparseMatrixA_bitmapP6__halfiiiiiiiiPS0_PPiS3_S3_PPmRi,
 * csrc/SpMM_API.cuh:112-120), for callers compiled against the reference.
 * Declared when <hip/hip_fp16.h> was included first.
 */
int InitSparseMatrixA_bitmap(__half* A_h, int M, int K, int tile_M, int tile_M_median, int tile_M_global, int tile_K,
                             int tile_K_median, int tile_K_global, __half** Compressed_Val, int** TileOffsets,
                             int** TileOffsets_median, int** TileOffsets_global, uint64_t** bitmap,
                             int& max_nnz_count);
#endif
#endif /* __cplusplus */

#endif /* SPMM_API_H */
