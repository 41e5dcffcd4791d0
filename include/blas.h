// blas::blas_init / blas::blas_destroy, the set-up hooks of the reference harness
// (include/blas.h:19-50; called from tests/includes/test_config.h:208,298).  The reference
// creates a vendor BLAS handle in a header-defined global (an ODR hazard when included
// twice); here the handle is the library's own context and everything is `inline`.
#pragma once
#include "common.h"
#include "qgemm.h"

// status of the last qgemm_init() on this handle; QGEMM_OK after a successful blas_init
using blas_handle_t = int;

namespace blas {

inline blas_handle_t blas_handle = QGEMM_ERR_NO_DEVICE;

inline void blas_init(blas_handle_t &handle) { handle = qgemm_init(); }
inline void blas_init() { blas_init(blas_handle); }
inline void blas_destroy(blas_handle_t &handle) {
    (void)qgemm_shutdown();
    handle = QGEMM_ERR_NO_DEVICE;
}
inline void blas_destroy() { blas_destroy(blas_handle); }

}  // namespace blas
