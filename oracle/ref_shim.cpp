/*
 * TEST INFRASTRUCTURE ONLY.  C-linkage door onto the reference's own
 * Tiled-CSL encoder, whose symbol is C++-mangled (declaration:
 * build/SpMM_API.cuh:55-62 of the reference).  The encoder itself is compiled
 * by oracle/Makefile straight from the reference checkout; this file holds
 * none of it.
 */
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdlib.h>

int InitSparseMatrixA_API(half* A_h, int M, int N, int K, uint32_t** Compressed_A, int** TileOffsets);
int InitSparseMatrixA_API_NoReorder(half* A_h, int M, int N, int K, uint32_t** Compressed_A, int** TileOffsets);

extern "C" int ref_InitSparseMatrixA_API(uint16_t* A_h, int M, int N, int K, uint32_t** Compressed_A,
                                         int** TileOffsets)
{
    return InitSparseMatrixA_API(reinterpret_cast<half*>(A_h), M, N, K, Compressed_A, TileOffsets);
}

extern "C" int ref_InitSparseMatrixA_API_NoReorder(uint16_t* A_h, int M, int N, int K, uint32_t** Compressed_A,
                                                   int** TileOffsets)
{
    return InitSparseMatrixA_API_NoReorder(reinterpret_cast<half*>(A_h), M, N, K, Compressed_A, TileOffsets);
}

extern "C" void ref_free(void* p)
{
    free(p);
}
