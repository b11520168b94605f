// Upload-time re-layout: GGUF block bytes -> the device-private planes described in formats.h.
//
// GGUF rows are arrays of packed blocks (/root/reference/fs/ggml/gguf.go:281-308 hands them out
// unchanged).  18-, 34- and 210-byte blocks are only 2-byte aligned, so a wavefront cannot read them
// with aligned 16-byte loads; splitting each block's fields into separate planes restores that.
// Runs once per tensor at load; every field offset and size is even, so the copy moves 16-bit units.
#include "internal.h"

namespace miqmm {

namespace {

// one thread per 16-bit unit of the source
template <int TYPE>
__global__ void relayout_kernel(const uint16_t *__restrict__ src, int64_t nblocks, uint16_t *__restrict__ p0,
                                uint16_t *__restrict__ p1, uint16_t *__restrict__ p2,
                                uint16_t *__restrict__ d) {
    constexpr int UNITS = (TYPE == T_Q4_0 ? Q4_0_BYTES : TYPE == T_Q8_0 ? Q8_0_BYTES : Q6_K_BYTES) / 2;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nblocks * UNITS) return;
    const int64_t blk = i / UNITS;
    const int u = (int)(i - blk * UNITS);
    const uint16_t v = src[i];
    if (TYPE == T_Q4_0) {  // d(1 unit) qs(8 units)
        if (u == 0) d[blk] = v; else p0[blk * 8 + (u - 1)] = v;
    } else if (TYPE == T_Q8_0) {  // d(1) qs(16)
        if (u == 0) d[blk] = v; else p0[blk * 16 + (u - 1)] = v;
    } else {  // Q6_K: ql(64) qh(32) scales(8) d(1)
        if (u < 64) p0[blk * 64 + u] = v;
        else if (u < 96) p1[blk * 32 + (u - 64)] = v;
        else if (u < 104) p2[blk * 8 + (u - 96)] = v;
        else d[blk] = v;
    }
}

}  // namespace

hipError_t launch_relayout(int type, const uint8_t *gguf, int64_t K, int64_t M, uint8_t *p0, uint8_t *p1,
                           uint8_t *p2, uint16_t *d, hipStream_t s) {
    if (K * M == 0) return hipSuccess;
    const uint16_t *src = (const uint16_t *)gguf;
    if (type == T_Q4_K) {
        return hipMemcpyAsync(p0, gguf, (size_t)(M * (K / QKK) * Q4_K_BYTES), hipMemcpyDeviceToDevice, s);
    } else if (type == T_Q4_0) {
        const int64_t nb = M * (K / QK), n = nb * (Q4_0_BYTES / 2);
        relayout_kernel<T_Q4_0><<<(unsigned)((n + 255) / 256), 256, 0, s>>>(src, nb, (uint16_t *)p0, nullptr, nullptr, d);
    } else if (type == T_Q8_0) {
        const int64_t nb = M * (K / QK), n = nb * (Q8_0_BYTES / 2);
        relayout_kernel<T_Q8_0><<<(unsigned)((n + 255) / 256), 256, 0, s>>>(src, nb, (uint16_t *)p0, nullptr, nullptr, d);
    } else if (type == T_Q6_K) {
        const int64_t nb = M * (K / QKK), n = nb * (Q6_K_BYTES / 2);
        relayout_kernel<T_Q6_K><<<(unsigned)((n + 255) / 256), 256, 0, s>>>(src, nb, (uint16_t *)p0, (uint16_t *)p1,
                                                                            (uint16_t *)p2, d);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace miqmm
