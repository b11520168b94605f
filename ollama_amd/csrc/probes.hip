// Measurement aids for bench_probes.py, not part of the product library: small kernels that each answer one
// question about this machine on which a design decision of the product kernels rests.
//   mi_probe_empty      what does a kernel launch cost when the kernel does nothing?
//   mi_probe_lds_b128   which lanes does the LDS serve together on a 16-byte read (which layouts are conflict-free)?
//   mi_probe_lane_map   how fast does a launch stream a matrix when the lanes of a 16-byte load are laid over the rows
//                       in different orders (what the address coalescer makes of each)?
//   mi_probe_flood_read what does a launch that requests all of its 66 MB at once achieve, row-strided or contiguous?
//   mi_probe_copy_stream  what does the stream of direct-to-LDS copies of a staged small-batch kernel cost by itself,
//                       and which of its copies cost what (bytes moved, or cache lines named)?
//   mi_probe_handoff    what does it cost to hand a partial tile from one workgroup to another inside a launch
//                       without device-scope fences (write-through stores, a flag, bypassing loads)?
// Every kernel exits on its own: the only waits on another workgroup are bounded polls.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef unsigned u4v __attribute__((ext_vector_type(4)));
typedef float f4v __attribute__((ext_vector_type(4)));

__global__ void empty_kernel() {}

// ---- LDS: `waves` waves (1..4, one per SIMD) that all do `iters` reads of 16 bytes per lane at lds[off[lane]], twelve
// in flight per wave; cycles of wave 0's loop to out[0], reads per wave to out[1].  One wave alone is bound by the
// latency of its reads, four keep the LDS busy.  The offsets come from the host, so any hypothesis about how lanes
// are grouped can be put to the counter SQ_LDS_BANK_CONFLICT and to the clock.
__global__ __launch_bounds__(256) void lds_b128_kernel(const int *__restrict__ off, int iters, long long *__restrict__ out) {
    __shared__ __attribute__((aligned(1024))) uint8_t lds[16384];
    const int lane = threadIdx.x & 63;
    for (int i = threadIdx.x; i < 16384 / 4; i += blockDim.x) reinterpret_cast<unsigned *>(lds)[i] = i * 2654435761u;
    __syncthreads();
    const unsigned o = (unsigned)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds + (unsigned)(off[lane] & 16368);
    u4v acc = {0, 0, 0, 0};
    __syncthreads();
    const long long c0 = clock64();
    for (int i = 0; i < iters; i += 12) {
        u4v v[12];
#pragma unroll
        for (int u = 0; u < 12; u++) asm volatile("ds_read_b128 %0, %1" : "=v"(v[u]) : "v"(o));
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]), "+v"(v[8]), "+v"(v[9]),
                       "+v"(v[10]), "+v"(v[11]));
#pragma unroll
        for (int u = 0; u < 12; u++) acc ^= v[u];
    }
    const long long c1 = clock64();
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) out[2] = 1;  // keeps the reads alive
    if (threadIdx.x == 0) { out[0] = c1 - c0; out[1] = (iters + 11) / 12 * 12; }
}

// ---- lane order of 16-byte global loads over a matrix of 144-byte records (the Q4_K super-block), 16 rows per
// wave-step, the row pitch a whole number of records.  Each step a wave reads the 128 quant bytes of four records of 16
// rows (eight loads of 16 bytes per lane in flight); what differs is which lane reads which piece:
//   mode 0  lane = row + 16 * piece   (the order an MFMA B operand wants: 16 rows apart between neighbouring lanes)
//   mode 1  lane = 4 * row + piece    (quads of lanes on 64 contiguous bytes)
//   mode 2  linear: lane l reads bytes 16 l .. of a contiguous 2 KiB (no rows at all: the reference line)
//   mode 3  lane = 8 * row + piece    (eight lanes on the 128 contiguous quant bytes of a row, eight rows per load)
template <int MODE>
__global__ __launch_bounds__(256) void lane_map_kernel(const uint8_t *__restrict__ p, int64_t pitch, int nsb, int groups, unsigned *__restrict__ out) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int waves_all = gridDim.x * 4, w = blockIdx.x * 4 + wave;
    u4v acc = {0, 0, 0, 0};
    for (int g = w; g < groups; g += waves_all) {
        const uint8_t *base = p + (int64_t)g * 16 * pitch;
        int64_t o;
        if (MODE == 0) o = (int64_t)(lane & 15) * pitch + 16 + 16 * (lane >> 4);
        else if (MODE == 1) o = (int64_t)(lane >> 2) * pitch + 16 + 16 * (lane & 3);
        else if (MODE == 3) o = (int64_t)(lane >> 3) * pitch + 16 + 16 * (lane & 7);
        else o = 16 * lane;
        for (int sb = 0; sb < nsb; sb += 4) {
            u4v v[8];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int64_t so = MODE == 2 ? (int64_t)(sb + u) * 2048 : (int64_t)(sb + u) * 144;
                v[2 * u] = *reinterpret_cast<const u4v *>(base + o + so);
                v[2 * u + 1] = *reinterpret_cast<const u4v *>(base + o + so + (MODE == 2 ? 1024 : MODE == 3 ? 8 * pitch : 64));
            }
#pragma unroll
            for (int u = 0; u < 8; u++) acc ^= v[u];
        }
    }
    unsigned x = acc.x ^ acc.y ^ acc.z ^ acc.w;
    for (int m = 1; m < 64; m <<= 1) x ^= __shfl_xor(x, m, 64);
    if (lane == 0) atomicXor(out + (blockIdx.x & 255), x);
}

// ---- everything in flight at once: the read pattern of the deep direct-load kernel on its gate + up launch, by itself.
// One workgroup of 14 waves per CU; a workgroup owns 7 consecutive groups of 16 rows (36,864 contiguous bytes each at
// K = 4096), two waves per group.  Every wave requests its whole share -- 18,432 bytes, 18 loads of 16 bytes per lane --
// before it looks at any of it:
//   mode 0  as the kernel does: wave h of a group takes the K half h of all 16 rows; per load a quad of lanes reads 64
//           contiguous bytes of a row, the 16 quads 16 different rows
//   mode 1  the same bytes of the matrix split the other way: wave h takes rows 8h .. 8h+7 whole, a contiguous run of
//           18,432 bytes, 1 KiB per load
template <int MODE>
__global__ __launch_bounds__(896) void flood_read_kernel(const uint8_t *__restrict__ p, int groups, unsigned *__restrict__ out) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = blockIdx.x * 7 + (wave >> 1), h = wave & 1;
    u4v acc = {0, 0, 0, 0};
    if (g < groups) {
        const uint8_t *base = p + (int64_t)g * 36864;
        u4v v[18];
        if (MODE == 0) {
            const uint8_t *q = base + (lane >> 2) * 2304 + h * 1152 + 16 * (lane & 3);
#pragma unroll
            for (int u = 0; u < 18; u++) v[u] = *reinterpret_cast<const u4v *>(q + 64 * u);
        } else {
            const uint8_t *q = base + h * 18432 + 16 * lane;
#pragma unroll
            for (int u = 0; u < 18; u++) v[u] = *reinterpret_cast<const u4v *>(q + 1024 * u);
        }
#pragma unroll
        for (int u = 0; u < 18; u++) acc ^= v[u];
    }
    unsigned x = acc.x ^ acc.y ^ acc.z ^ acc.w;
    for (int m = 1; m < 64; m <<= 1) x ^= __shfl_xor(x, m, 64);
    if (lane == 0) atomicXor(out + (blockIdx.x & 255), x);
}

// ---- the copy stream of a staged small-batch kernel, by itself.  A wave owns groups of 16 rows of a Q6_K-like
// matrix (per row and super-block: 128 B of low quant bits, 64 B of high bits, 16 B of sub-block scales, 2 B of a
// super-block scale, each in a plane of its own) and per super-block copies them into its LDS stage with
// direct-to-LDS loads, together with the activations of that super-block (2 KiB of quants, 256 B of digits, 32 B of
// scales: the same for every row group, so always cache hits).  No arithmetic.  `mask` leaves copies out:
//   bit 0 low bits (2 copies)  1 high bits (1)  2 sub-block scales (1: sixteen 16-byte pieces, each from its own line)
//   bit 3 super-block scales (1: sixteen 2-byte pieces)  4 activation quants (2)  5 digits and activation scales (2)
__device__ __forceinline__ void dma_lds16(const uint8_t *base, unsigned off, unsigned lds_addr) {
    const unsigned long long v = (unsigned long long)base;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
    const uint8_t *b = (const uint8_t *)(((unsigned long long)hi << 32) | lo);
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(b), "s"(lds_addr) : "memory");
}
__device__ __forceinline__ void dma_lds4(const uint8_t *base, unsigned off, unsigned lds_addr) {
    const unsigned long long v = (unsigned long long)base;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
    const uint8_t *b = (const uint8_t *)(((unsigned long long)hi << 32) | lo);
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1" ::"v"(off), "s"(b), "s"(lds_addr) : "memory");
}

struct CopyArgs {
    const uint8_t *ql, *qh, *sc, *d, *aq, *ad;  // planes: [rows][nsb*128], [rows][nsb*64], [rows][nsb*16], [rows][nsb*2]; act [nsb*2048], [nsb*512]
    int nsb, groups, mask;
};

__global__ __launch_bounds__(128) void copy_stream_kernel(CopyArgs a, unsigned *__restrict__ out) {
    __shared__ __attribute__((aligned(1024))) uint8_t lds[2 * 2 * 8192];  // two waves, two stages of 8 KiB
    const unsigned lbase = (unsigned)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves_all = gridDim.x * 2, w = blockIdx.x * 2 + wave;
    const int row = lane >> 2, pc = lane & 3;  // 16 rows x 4 pieces of 16 bytes per copy instruction
    unsigned acc = 0;
    const int ncopy = 2 * (a.mask & 1) + ((a.mask >> 1) & 1) + ((a.mask >> 2) & 1) + ((a.mask >> 3) & 1) + 2 * ((a.mask >> 4) & 1) + 2 * ((a.mask >> 5) & 1);
    for (int g = w; g < a.groups; g += waves_all) {
        const int64_t r0 = (int64_t)g * 16;
        for (int sb = 0; sb < a.nsb; sb++) {
            const unsigned st = lbase + (wave * 2 + (sb & 1)) * 8192;
            if (a.mask & 1) {
                dma_lds16(a.ql + (r0 * a.nsb + sb) * 128, (unsigned)(row * a.nsb * 128 + 16 * pc), st);
                dma_lds16(a.ql + (r0 * a.nsb + sb) * 128 + 64, (unsigned)(row * a.nsb * 128 + 16 * pc), st + 1024);
            }
            if (a.mask & 2) dma_lds16(a.qh + (r0 * a.nsb + sb) * 64, (unsigned)(row * a.nsb * 64 + 16 * pc), st + 2048);
            if (a.mask & 4) dma_lds16(a.sc + (r0 * a.nsb + sb) * 16, (unsigned)((lane & 15) * a.nsb * 16), st + 3072);
            if (a.mask & 8) dma_lds4(a.d, (unsigned)(((r0 + (lane & 15)) * a.nsb + sb) * 2) & ~3u, st + 4096);  // the dword holding the 2 bytes
            if (a.mask & 16) {
                dma_lds16(a.aq + (int64_t)sb * 2048, 16u * lane, st + 4352);
                dma_lds16(a.aq + (int64_t)sb * 2048 + 1024, 16u * lane, st + 5376);
            }
            if (a.mask & 32) {
                dma_lds4(a.ad + (int64_t)sb * 512, 4u * lane, st + 6400);
                dma_lds4(a.ad + (int64_t)sb * 512 + 256, 4u * lane, st + 6656);
            }
            // the other stage (filled one super-block ago) must have landed -- this super-block's ncopy copies stay in
            // flight -- and is read, as a kernel's multiply would, before the next round overwrites it
            switch (ncopy) {
            case 0: case 1: asm volatile("s_waitcnt vmcnt(1)" ::: "memory"); break;
            case 2: asm volatile("s_waitcnt vmcnt(2)" ::: "memory"); break;
            case 3: asm volatile("s_waitcnt vmcnt(3)" ::: "memory"); break;
            case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
            case 5: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
            case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
            case 7: asm volatile("s_waitcnt vmcnt(7)" ::: "memory"); break;
            case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
            default: asm volatile("s_waitcnt vmcnt(9)" ::: "memory"); break;
            }
            acc ^= *reinterpret_cast<const volatile unsigned *>(lds + (wave * 2 + ((sb + 1) & 1)) * 8192 + 4 * lane);
        }
    }
    for (int m = 1; m < 64; m <<= 1) acc ^= __shfl_xor(acc, m, 64);
    if (lane == 0) atomicXor(out + (blockIdx.x & 255), acc);
}

// ---- hand-off of partial tiles between workgroups of one launch, without fences.  tiles x 4 workgroups; workgroup
// (s, t) holds the partial plane s of tile t: 128 values per thread (a tile of 128 KiB), here simply s + 1.  With hops == 0 every
// workgroup writes its partial to part[s][t] and is done.  With hops == 2: slices 0 and 2 write theirs with
// write-through stores, wait for the stores and raise flag[s][t]; slice 1 polls flag 0, reads partial 0 with
// cache-bypassing loads, adds its own, writes the sum and raises flag 1; slice 3 does the same with partial 2 and then
// with the sum of slice 1, and writes the total (10 everywhere) to y.  Workgroups are numbered slice-major, so a
// consumer is dispatched after its producers; every poll is bounded (err[0] counts polls that ran out).
__device__ __forceinline__ bool poll(const unsigned *flag, unsigned want, int limit) {
    for (int i = 0; i < limit; i++) {
        if (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) == want) return true;
        __builtin_amdgcn_s_sleep(2);
    }
    return false;
}

__global__ __launch_bounds__(256) void handoff_kernel(float *__restrict__ part, unsigned *__restrict__ flag, float *__restrict__ y,
                                                      unsigned *__restrict__ err, int tiles, int hops, unsigned epoch, int limit) {
    constexpr int words = 128;  // per thread: a tile of 128 KiB
    const int s = blockIdx.x / tiles, t = blockIdx.x % tiles, tid = threadIdx.x;
    const int64_t tile_words = (int64_t)words * 256;
    float *mine = part + ((int64_t)s * tiles + t) * tile_words;
    const float own = (float)(s + 1);
    if (hops == 0) {
#pragma unroll 8
        for (int i = 0; i < words; i += 4) *reinterpret_cast<f4v *>(mine + ((int64_t)(i / 4) * 256 + tid) * 4) = (f4v){own, own, own, own};
        return;
    }
    __shared__ int ok;
    auto take = [&](int from, float *sum) {  // sum[i] += partial `from` of this tile, once its flag is up
        if (tid == 0) ok = poll(flag + from * tiles + t, epoch, limit) ? 1 : 0;
        __syncthreads();
        const bool good = ok != 0;
        __syncthreads();
        if (!good) {
            if (tid == 0) atomicAdd(err, 1u);
            return;
        }
        const float *src = part + ((int64_t)from * tiles + t) * tile_words;
#pragma unroll
        for (int i = 0; i < words; i += 16) {  // system-scope loads of 16 bytes (they bypass the caches), four in flight
            f4v v[4];
#pragma unroll
            for (int u = 0; u < 4; u++) asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1" : "=v"(v[u]) : "v"(src + ((int64_t)(i / 4 + u) * 256 + tid) * 4) : "memory");
            asm volatile("s_waitcnt vmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3])::"memory");
#pragma unroll
            for (int u = 0; u < 4; u++) { sum[i + 4 * u] += v[u].x; sum[i + 4 * u + 1] += v[u].y; sum[i + 4 * u + 2] += v[u].z; sum[i + 4 * u + 3] += v[u].w; }
        }
    };
    auto give = [&](const float *sum) {  // write-through stores, wait for them, then the flag
#pragma unroll
        for (int i = 0; i < words; i += 4) {  // system-scope (write-through) stores of 16 bytes
            const f4v v = {sum[i], sum[i + 1], sum[i + 2], sum[i + 3]};
            asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(mine + ((int64_t)(i / 4) * 256 + tid) * 4), "v"(v) : "memory");
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) __hip_atomic_store(flag + s * tiles + t, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    };
    float sum[words];
#pragma unroll
    for (int i = 0; i < words; i++) sum[i] = own;
    if (s == 0 || s == 2) {
        give(sum);
    } else if (s == 1) {
        take(0, sum);
        give(sum);
    } else {
        take(2, sum);
        take(1, sum);
#pragma unroll
        for (int i = 0; i < words; i += 4)
            *reinterpret_cast<f4v *>(y + (int64_t)t * tile_words + ((int64_t)(i / 4) * 256 + tid) * 4) = (f4v){sum[i], sum[i + 1], sum[i + 2], sum[i + 3]};
    }
}

}  // namespace

extern "C" {

// one empty launch of `blocks` workgroups of `threads`
int mi_probe_empty(int blocks, int threads, void *stream) {
    if (blocks < 1 || threads < 1 || threads > 1024) return -1;
    empty_kernel<<<blocks, threads, 0, (hipStream_t)stream>>>();
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

// off: device, 64 byte offsets (multiples of 16, below 16384); out: device, three int64 (cycles, reads, scratch)
int mi_probe_lds_b128(const int *off, int iters, int waves, long long *out, void *stream) {
    if (!off || !out || iters < 1 || waves < 1 || waves > 4) return -1;
    lds_b128_kernel<<<1, 64 * waves, 0, (hipStream_t)stream>>>(off, iters, out);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

// p: device buffer of rows * pitch bytes (pitch = nsb * 144; mode 2 reads it as groups * nsb * 2048 contiguous bytes and
// needs that much); rows a multiple of 16; nsb a multiple of 4; out: device scratch of 256 words
int mi_probe_lane_map(int mode, const void *p, int64_t rows, int nsb, int blocks, unsigned *out, void *stream) {
    if (!p || !out || rows < 16 || rows % 16 || nsb < 4 || nsb % 4 || blocks < 1 || mode < 0 || mode > 3) return -1;
    hipStream_t s = (hipStream_t)stream;
    const uint8_t *q = (const uint8_t *)p;
    const int64_t pitch = (int64_t)nsb * 144;
    const int groups = (int)(rows / 16);
    if (mode == 0) lane_map_kernel<0><<<blocks, 256, 0, s>>>(q, pitch, nsb, groups, out);
    else if (mode == 1) lane_map_kernel<1><<<blocks, 256, 0, s>>>(q, pitch, nsb, groups, out);
    else if (mode == 3) lane_map_kernel<3><<<blocks, 256, 0, s>>>(q, pitch, nsb, groups, out);
    else lane_map_kernel<2><<<blocks, 256, 0, s>>>(q, pitch, nsb, groups, out);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

// p: device buffer of groups * 36864 bytes (groups of 16 rows of 2304 bytes); out: device scratch of 256 words
int mi_probe_flood_read(int mode, const void *p, int groups, unsigned *out, void *stream) {
    if (!p || !out || groups < 1 || mode < 0 || mode > 1) return -1;
    const int blocks = (groups + 6) / 7;
    if (mode == 0) flood_read_kernel<0><<<blocks, 896, 0, (hipStream_t)stream>>>((const uint8_t *)p, groups, out);
    else flood_read_kernel<1><<<blocks, 896, 0, (hipStream_t)stream>>>((const uint8_t *)p, groups, out);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

// planes: device buffers of rows * nsb * {128, 64, 16, 2} bytes and activations of nsb * {2048, 512} bytes; rows a
// multiple of 16, rows * nsb * 128 below 4 GiB per 16-row group offset (32-bit lane offsets: nsb * 128 * 16 < 2^32)
int mi_probe_copy_stream(const void *ql, const void *qh, const void *sc, const void *d, const void *aq, const void *ad, int64_t rows,
                         int nsb, int mask, int blocks, unsigned *out, void *stream) {
    if (!ql || !qh || !sc || !d || !aq || !ad || !out || rows < 16 || rows % 16 || nsb < 1 || nsb > 4096 || blocks < 1) return -1;
    CopyArgs a{(const uint8_t *)ql, (const uint8_t *)qh, (const uint8_t *)sc, (const uint8_t *)d, (const uint8_t *)aq, (const uint8_t *)ad,
               nsb, (int)(rows / 16), mask};
    copy_stream_kernel<<<blocks, 128, 0, (hipStream_t)stream>>>(a, out);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

// part: device, 4 * tiles * 32768 floats; flag: device, 4 * tiles words (zero before the first call; pass a new
// epoch > 0 per call instead of clearing); y: device, tiles * 32768 floats; err: device word, zero before.
// tiles * 4 workgroups must all be resident at once (tiles <= a quarter of the CUs); hops 0 or 2.
int mi_probe_handoff(float *part, unsigned *flag, float *y, unsigned *err, int tiles, int hops, unsigned epoch, int poll_limit, void *stream) {
    if (!part || !flag || !y || !err || tiles < 1 || tiles > 64 || (hops != 0 && hops != 2) || !epoch || poll_limit < 1) return -1;
    handoff_kernel<<<4 * tiles, 256, 0, (hipStream_t)stream>>>(part, flag, y, err, tiles, hops, epoch, poll_limit);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

}  // extern "C"
