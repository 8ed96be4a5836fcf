/*
 * TEST INFRASTRUCTURE ONLY.  C-linkage doors onto the reference's own
 * Tiled-CSL encoder (declaration: build/SpMM_API.cuh:55-62 of the reference) and
 * its 2:4 + residual split (kernel_benchmark/spmm_decompose.h:12), whose symbols
 * are C++-mangled.  Both are compiled by oracle/Makefile straight from the
 * reference checkout; this file holds none of them.
 */
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdlib.h>

int InitSparseMatrixA_API(half* A_h, int M, int N, int K, uint32_t** Compressed_A, int** TileOffsets);
int InitSparseMatrixA_API_NoReorder(half* A_h, int M, int N, int K, uint32_t** Compressed_A, int** TileOffsets);
void decompose(half* A, half* A1, half* A2, int length);

extern "C" void ref_decompose(uint16_t* A, uint16_t* A1, uint16_t* A2, int length)
{
    decompose(reinterpret_cast<half*>(A), reinterpret_cast<half*>(A1), reinterpret_cast<half*>(A2), length);
}

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
