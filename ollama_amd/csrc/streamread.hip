// Measurement aid for bench.py, not part of the product library: how fast can ONE kernel launch read N
// bytes from HBM on this machine?  A grid of workgroups streams the buffer with 16-byte loads, several in
// flight per lane, folds what it read into one word per workgroup (so the loads cannot be dropped) and
// stores that.  bench.py times it back to back over rotating buffers, like the GEMV launches, and takes
// the best of a few grid shapes: the launch-inclusive bandwidth a pure read of that size reaches is the
// practical ceiling next to which the GEMV's own figure is shown.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

template <int UNROLL>
__global__ __launch_bounds__(1024) void stream_read_kernel(const uint4 *__restrict__ p, int64_t n16, unsigned *__restrict__ out) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint4 acc = make_uint4(0, 0, 0, 0);
    for (; i + (UNROLL - 1) * stride < n16; i += UNROLL * stride) {
        uint4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) v[u] = p[i + u * stride];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) { acc.x ^= v[u].x; acc.y ^= v[u].y; acc.z ^= v[u].z; acc.w ^= v[u].w; }
    }
    for (; i < n16; i += stride) { const uint4 v = p[i]; acc.x ^= v.x; acc.y ^= v.y; acc.z ^= v.z; acc.w ^= v.w; }
    unsigned w = acc.x ^ acc.y ^ acc.z ^ acc.w;
    for (int m = 1; m < 64; m <<= 1) w ^= __shfl_xor(w, m, 64);
    if ((threadIdx.x & 63) == 0) atomicXor(out + blockIdx.x, w);
}

}  // namespace

// Queues one read of `bytes` (a multiple of 16) from device memory p on `stream` with `blocks` workgroups of
// `threads` (a multiple of 64, at most 1024) and `unroll` (1, 2, 4 or 8) loads in flight per lane; out: device
// scratch of `blocks` words.
extern "C" int mi_stream_read(const void *p, int64_t bytes, int blocks, int threads, int unroll, unsigned *out, void *stream) {
    if (!p || !out || bytes < 16 || bytes % 16 || blocks < 1 || threads < 64 || threads > 1024 || threads % 64) return -1;
    hipStream_t s = (hipStream_t)stream;
    const uint4 *q = (const uint4 *)p;
    const int64_t n16 = bytes / 16;
    switch (unroll) {
    case 1: stream_read_kernel<1><<<blocks, threads, 0, s>>>(q, n16, out); break;
    case 2: stream_read_kernel<2><<<blocks, threads, 0, s>>>(q, n16, out); break;
    case 4: stream_read_kernel<4><<<blocks, threads, 0, s>>>(q, n16, out); break;
    case 8: stream_read_kernel<8><<<blocks, threads, 0, s>>>(q, n16, out); break;
    default: return -1;
    }
    return hipGetLastError() == hipSuccess ? 0 : -2;
}
