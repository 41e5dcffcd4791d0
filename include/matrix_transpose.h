// matrix_transpose<T>(idata, odata, M, N): odata[n*M + m] = idata[m*N + n].
// Same declaration as the reference's src/include/matrix_transpose.h:3-4 (defined in
// src/transpose/transpose.cu:60-74 for 2-byte T with M % 64 == 0, N % 32 == 0); here any M, N
// and 1-, 2- or 4-byte T.  Other sizes print to std::cerr and return, like the reference.
#pragma once
#include "common.h"
#include "qgemm.h"

template <typename T>
inline void matrix_transpose(const T *idata, T *odata, int M, int N) {
    if constexpr (sizeof(T) == 1 || sizeof(T) == 2 || sizeof(T) == 4) {
        const int st = qgemm_transpose((int)sizeof(T), idata, odata, (size_t)M, (size_t)N, nullptr);
        if (st != QGEMM_OK) std::cerr << "matrix_transpose: " << qgemm_status_string(st) << std::endl;
    } else {
        std::cerr << "Only support 1-, 2- and 4-byte data types now." << std::endl;
    }
}
