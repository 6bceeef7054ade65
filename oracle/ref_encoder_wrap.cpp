// Wrapper translation unit for building the reference's own host encoder as a
// checker.  TEST INFRASTRUCTURE ONLY: the text of the reference function is
// never stored in this repository; the Makefile beside this file extracts it
// from the reference tree at build time into a temporary include
// (REF_ENCODER_INC) that is deleted again once the object is built.
//
// The reference function (csrc/SpMM_API.cuh:112-241) needs only `half`,
// `__half2float`, `__float2half`, `__host__`, <vector> and malloc/realloc;
// the ROCm headers already in the image provide the first four on the host.
#include <cstdint>
#include <cstdlib>
#include <vector>
#include <hip/hip_runtime_api.h>
#include <hip/hip_fp16.h>

#ifndef __host__
#define __host__
#endif
typedef __half half;

#include REF_ENCODER_INC

extern "C" int ref_InitSparseMatrixA_bitmap(uint16_t* A_h, int M, int K, uint16_t** Compressed_Val,
                                            int** TileOffsets, int** TileOffsets_median,
                                            int** TileOffsets_global, uint64_t** bitmap, int* max_nnz_count)
{
    static_assert(sizeof(half) == sizeof(uint16_t), "half must be 2 bytes");
    int  max_nnz = 0;
    half* vals   = nullptr;
    int  g       = InitSparseMatrixA_bitmap(reinterpret_cast<half*>(A_h), M, K, 8, 16, 64, 8, 64, 64, &vals,
                                            TileOffsets, TileOffsets_median, TileOffsets_global, bitmap, max_nnz);
    *Compressed_Val = reinterpret_cast<uint16_t*>(vals);
    *max_nnz_count  = max_nnz;
    return g;
}

extern "C" void ref_free(void* p)
{
    free(p);
}
