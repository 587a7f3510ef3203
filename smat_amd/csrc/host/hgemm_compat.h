// Source-level compatibility with the reference's kernel entry point, so a
// `Tester`-style caller compiles unchanged against this library:
//   HGEMM_FUNC_SPARSE2(mmaCBTKernel)            src/cuda_hgemm/src/main.cu:7,19
//   void mmaCBTKernel(half*, int*, int*, half*, half*, size_t, size_t, size_t,
//                     size_t, int*, int*)       src/cuda_hgemm/src/mma/mmaCBT.cu:83-88
// `half` is the 16-bit storage type here (the host never does arithmetic on it).
// Failures end the process the way HGEMM_CHECK_* does (common/common.h:21-27).
#pragma once
#include <cstdint>
#include <cstdio>
#include <cstdlib>

#include "../../../include/smat.h"

#ifndef SMAT_HALF_DEFINED
#define SMAT_HALF_DEFINED
typedef uint16_t half;
#endif

#define HLOG(format, ...) fprintf(stderr, "[SMAT %s:%d] " format "\n", __FILE__, __LINE__, ##__VA_ARGS__)
#define SMAT_CHECK(call)                                                            \
    do {                                                                            \
        int rc_ = (call);                                                           \
        if (rc_ != SMAT_OK) {                                                       \
            HLOG("%s failed (%d): %s", #call, rc_, smat_last_error());              \
            exit(EXIT_FAILURE);                                                     \
        }                                                                           \
    } while (0)

inline void mmaCBTKernel(half *bcsrValuesA, int *bcsrRowPtrA, int *bcsrColIdxA, half *B, half *C, size_t M,
                         size_t N, size_t K, size_t nonzeroBlocks, int *blockInfo,
                         int *relativeBlockIndexMapping)
{
    SMAT_CHECK(smat_spmm_bcsr_f16(bcsrValuesA, bcsrRowPtrA, bcsrColIdxA, B, C, M, N, K, nonzeroBlocks, blockInfo,
                                  relativeBlockIndexMapping));
}
