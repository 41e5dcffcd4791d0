// Probes of the hardware behaviour the GEMM kernels are built on.  The gfx950
// counterpart of the reference's playground/ (ldmatrix / movmatrix lane-layout
// probes): each probe runs one wave and the host compares what came back with
// the layout the kernels assume.
#pragma once
#include "gemm_mfma.cuh"

namespace qgemm {

// One wave fetches 64 x 16 bytes from `src` with per-lane byte offsets `voff`
// through buffer_load_dwordx4 ... lds into LDS at `lds_base`, then copies the
// 1 KiB at lds_base back to `out`.  LDS is pre-filled with 0xA5 so "not written"
// and "written with zeros" can be told apart.  `range` is the buffer size: lanes
// whose offset lies beyond it are out of range.
__global__ void __launch_bounds__(64) probe_lds_dma_kernel(const char *src, const uint32_t *voff, uint32_t range,
                                                           uint32_t lds_base, uint32_t soffset, char *out) {
#if defined(__HIP_DEVICE_COMPILE__)
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const int lane = threadIdx.x;
    *(v4i *)(smem + lds_base + lane * 16) = v4i{(int)0xA5A5A5A5, (int)0xA5A5A5A5, (int)0xA5A5A5A5, (int)0xA5A5A5A5};
    __syncthreads();
    const __amdgpu_buffer_rsrc_t r = make_rsrc(src, range);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void *)(smem + lds_base), 16, voff[lane], soffset, 0, 0);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __syncthreads();
    *(v4i *)(out + lane * 16) = *(const v4i *)(smem + lds_base + lane * 16);
#endif
}

// One MFMA on operands taken verbatim from memory: lane l's first operand is the
// 32 bytes at x + 32*l, second operand at y + 32*l (the 16-byte MFMAs use the
// first 16 of each and then the second 16, exactly like mma128).  Accumulator
// registers go to out[4*l .. 4*l+3] (raw 32-bit).
template <int ARITH>
__global__ void __launch_bounds__(64) probe_mfma_kernel(const char *x, const char *y, int *out) {
#if defined(__HIP_DEVICE_COMPILE__)
    const int lane = threadIdx.x;
    const v4i x0 = *(const v4i *)(x + lane * 32), x1 = *(const v4i *)(x + lane * 32 + 16);
    const v4i y0 = *(const v4i *)(y + lane * 32), y1 = *(const v4i *)(y + lane * 32 + 16);
    typename AccT<ARITH>::type c = {0, 0, 0, 0};
    c = mma128<ARITH>(x0, x1, y0, y1, c);
    // (bit_cast of the whole vector: bit_cast of a single vector element reads element 0)
    *(v4i *)(out + lane * 4) = __builtin_bit_cast(v4i, c);
#endif
}

// Lane l loads 8 bytes at byte offset 4 * l of a raw buffer of `range` bytes (an a_scale row with an odd number of K
// blocks starts every other row at such an offset, and the last pair of the last row straddles the end of the range).
__global__ void __launch_bounds__(64) probe_b64_load_kernel(const float *src, uint32_t range, int *out) {
    const __amdgpu_buffer_rsrc_t r = make_rsrc(src, range);
    const int lane = threadIdx.x;
    const v2i v = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(r, lane * 4, 0, 0));
    out[2 * lane] = v[0];
    out[2 * lane + 1] = v[1];
}

// Every workgroup records which XCD (XCC_ID hardware register) and CU it ran on.
__global__ void __launch_bounds__(64) probe_xcc_kernel(uint32_t *out) {
#if defined(__HIP_DEVICE_COMPILE__)
    // s_getreg_b32 of HW_REG_XCC_ID (id 20), all 32 bits: XCC_ID in bits 3:0
    const uint32_t xcc = __builtin_amdgcn_s_getreg((31 << 11) | 20);
    // HW_REG_HW_ID (id 4): CU id in bits 11:8, SE id in bits 15:13 on gfx9
    const uint32_t hw = __builtin_amdgcn_s_getreg((31 << 11) | 4);
    if (threadIdx.x == 0) {
        out[blockIdx.x * 2] = xcc;
        out[blockIdx.x * 2 + 1] = hw;
    }
#endif
}

}  // namespace qgemm
