// Backend detection for the host API headers.  Same role as the reference's
// include/common.h:3-28; this build has one backend (HIP on gfx950).
#pragma once

#if defined(__HIPCC__) || defined(__HIP_PLATFORM_AMD__) || defined(QGEMM_USE_HIP)
#ifndef USE_HIP
#define USE_HIP
#endif
#endif

#ifndef USE_HIP
#error "qgemm host API: compile with hipcc (or define QGEMM_USE_HIP and add the HIP include path)"
#endif

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <iostream>
