// Plain copies with the access patterns of the two prefill kernels, and an empty launch: what this GPU does
// for a kernel that only moves the bytes.  Measurement aid of bench.py (a yardstick beside the 8 TB/s vendor
// peak), not part of the library: nothing in the package loads it.
//
//   copy_rows   every lane 16 bytes, a wave two vectors per lane = 2 KB of one row, streamed accesses:
//               the time-contiguous kernel without its arithmetic
//   copy_tiles  [B, L, rowbytes] memory in tiles of 32 rows x 512 bytes: 8 bytes per lane, 8 rows per wave (from 40 MB
//               of traffic: 16 rows x 512 bytes, 4 rows per wave, as the kernel's unmasked launches of that size),
//               4 waves per block, buffer accesses, consecutive time tiles of a column on one XCD, stores written
//               through from 64 MB of traffic: the channel-contiguous kernel without history, taps, LDS and arithmetic
//   copy_tile_shape  the same memory in other tile shapes (16 x 512 B, 16 x 1 KB and 32 x 1 KB with 16-byte lanes,
//               64 x 256 B with 16-byte lanes and four rows per instruction), blocks in address order: would another
//               decomposition of the channel-contiguous tensor stream faster?
//   empty_launch  a kernel of one wave that does nothing
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

__global__ __launch_bounds__(256) void copy_rows_kernel(const u32x4 *in, u32x4 *out, uint32_t nvec)
{
    const uint32_t wave = blockIdx.x * 4u + (threadIdx.x >> 6), lane = threadIdx.x & 63u;
    const uint32_t v0 = wave * 128u + lane, v1 = v0 + 64u;
    u32x4 a = {0, 0, 0, 0}, b = {0, 0, 0, 0};
    if (v0 < nvec) a = __builtin_nontemporal_load(in + v0);
    if (v1 < nvec) b = __builtin_nontemporal_load(in + v1);
    if (v0 < nvec) __builtin_nontemporal_store(a, out + v0);
    if (v1 < nvec) __builtin_nontemporal_store(b, out + v1);
}

struct Tiles {
    const char *in;
    char *out;
    uint32_t ncols, nct, ntt, L, rowbytes;
};
constexpr uint64_t kThroughBytes = 64ull << 20;   // traffic from which the channel-contiguous prefill writes its stores through
constexpr uint64_t kShortSlabBytes = 40ull << 20; // ... and from which its unmasked launches run slabs of four rows

template <int AUXS, uint32_t R> __global__ __launch_bounds__(256) void copy_tiles_kernel(const Tiles g)
{
    constexpr uint32_t WT = 4, VB = 8;
    // block = (column group * ntt + time tile) * 8 + XCD; column = (batch entry, channel tile)
    const uint32_t x = blockIdx.x & 7u, j = blockIdx.x >> 3;
    const uint32_t jg = j / g.ntt, tt = j - jg * g.ntt;
    const uint32_t q = jg * 8u + x;
    if (q >= g.ncols) return;
    const uint32_t b = q / g.nct, ct = q - b * g.nct;
    const uint32_t wt = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63u;
    const uint32_t cbase = ct * 64u * VB;
    const uint32_t t0 = (tt * WT + wt) * R;
    if (t0 >= g.L) return;
    const uint32_t width = g.rowbytes - cbase < 64u * VB ? g.rowbytes - cbase : 64u * VB;
    const uint32_t rows = g.L - t0 < R ? g.L - t0 : R;
    const size_t base = ((size_t)b * g.L + t0) * g.rowbytes + cbase;
    const uint32_t nrec = (rows - 1u) * g.rowbytes + width;   // rows past the end and lanes past the row: out of range
    __amdgpu_buffer_rsrc_t ri = __builtin_amdgcn_make_buffer_rsrc((void *)(g.in + base), 0, (int)nrec, 0x00020000);
    __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc((void *)(g.out + base), 0, (int)nrec, 0x00020000);
    const uint32_t voff = lane * VB < width ? lane * VB : 0x80000000u;
    u32x2 v[R];
#pragma unroll
    for (uint32_t r = 0; r < R; ++r) v[r] = __builtin_amdgcn_raw_buffer_load_b64(ri, (int)voff, (int)(r * g.rowbytes), 2);
#pragma unroll
    for (uint32_t r = 0; r < R; ++r) __builtin_amdgcn_raw_buffer_store_b64(v[r], ro, (int)voff, (int)(r * g.rowbytes), AUXS);
}

// Tiles of R * WT * (64 / LPR) rows x LPR * VB bytes: a lane moves VB bytes, LPR lanes cover one row of the tile, a
// load instruction 64 / LPR rows, a wave R instructions, a block WT waves.  Blocks in address order (channel tile
// fastest, then time tile, then batch entry); stores written through like the kernel's in large launches.
template <int VB, int R, int WT, int LPR>
__global__ __launch_bounds__(64 * WT) void copy_shape_kernel(const Tiles g)
{
    constexpr uint32_t RPI = 64 / LPR, WB = LPR * VB;           // rows per instruction, tile width in bytes
    const uint32_t ct = blockIdx.x % g.nct, r0 = blockIdx.x / g.nct, tt = r0 % g.ntt, b = r0 / g.ntt;
    const uint32_t wt = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63u;
    const uint32_t cbase = ct * WB;
    const uint32_t t0 = (tt * WT + wt) * R * RPI;
    if (t0 >= g.L) return;
    const uint32_t width = g.rowbytes - cbase < WB ? g.rowbytes - cbase : WB;
    const uint32_t rows = g.L - t0 < R * RPI ? g.L - t0 : R * RPI;
    const size_t base = ((size_t)b * g.L + t0) * g.rowbytes + cbase;
    const uint32_t nrec = (rows - 1u) * g.rowbytes + width;
    __amdgpu_buffer_rsrc_t ri = __builtin_amdgcn_make_buffer_rsrc((void *)(g.in + base), 0, (int)nrec, 0x00020000);
    __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc((void *)(g.out + base), 0, (int)nrec, 0x00020000);
    const uint32_t col = (lane % LPR) * VB;
    const uint32_t voff = col < width ? col + (lane / LPR) * g.rowbytes : 0x80000000u;
    if constexpr (VB == 8) {
        u32x2 v[R];
#pragma unroll
        for (uint32_t r = 0; r < R; ++r) v[r] = __builtin_amdgcn_raw_buffer_load_b64(ri, (int)voff, (int)(r * RPI * g.rowbytes), 2);
#pragma unroll
        for (uint32_t r = 0; r < R; ++r) __builtin_amdgcn_raw_buffer_store_b64(v[r], ro, (int)voff, (int)(r * RPI * g.rowbytes), 2 | 16);
    } else {
        u32x4 v[R];
#pragma unroll
        for (uint32_t r = 0; r < R; ++r) v[r] = __builtin_amdgcn_raw_buffer_load_b128(ri, (int)voff, (int)(r * RPI * g.rowbytes), 2);
#pragma unroll
        for (uint32_t r = 0; r < R; ++r) __builtin_amdgcn_raw_buffer_store_b128(v[r], ro, (int)voff, (int)(r * RPI * g.rowbytes), 2 | 16);
    }
}

template <int VB, int R, int WT, int LPR>
static int launch_shape(const void *in, void *out, uint32_t batch, uint32_t rows, uint32_t rowbytes, hipStream_t stream)
{
    Tiles g;
    g.in = (const char *)in;
    g.out = (char *)out;
    g.nct = (rowbytes + LPR * VB - 1) / (LPR * VB);
    g.ntt = (rows + R * WT * (64 / LPR) - 1) / (R * WT * (64 / LPR));
    g.L = rows;
    g.rowbytes = rowbytes;
    g.ncols = batch * g.nct;
    const uint64_t grid = (uint64_t)batch * g.nct * g.ntt;
    if (grid >= (1ull << 31)) return 1;
    hipLaunchKernelGGL((copy_shape_kernel<VB, R, WT, LPR>), dim3((uint32_t)grid), dim3(64 * WT), 0, stream, g);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

__global__ void empty_kernel() {}

extern "C" {

__attribute__((visibility("default"))) int copy_rows(const void *in, void *out, uint64_t bytes, void *stream)
{
    if (bytes % 16 || bytes / 16 >= (1ull << 32) || ((uintptr_t)in | (uintptr_t)out) % 16) return 1;
    const uint32_t nvec = (uint32_t)(bytes / 16);
    if (nvec == 0) return 0;
    const uint32_t nwaves = (nvec + 127u) / 128u;
    hipLaunchKernelGGL(copy_rows_kernel, dim3((nwaves + 3u) / 4u), dim3(256), 0, (hipStream_t)stream, (const u32x4 *)in,
                       (u32x4 *)out, nvec);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

__attribute__((visibility("default"))) int copy_tiles(const void *in, void *out, uint32_t batch, uint32_t rows, uint32_t rowbytes,
                                                      void *stream)
{
    if (rowbytes % 8 || ((uintptr_t)in | (uintptr_t)out) % 8 || batch == 0 || rows == 0 || rowbytes == 0) return 1;
    if ((uint64_t)rowbytes * 8 >= (1ull << 31)) return 1;   // rows are 32-bit offsets inside a wave's resource
    Tiles g;
    g.in = (const char *)in;
    g.out = (char *)out;
    g.nct = (rowbytes + 511u) / 512u;
    const uint64_t traffic = 2ull * batch * rows * rowbytes;
    const uint32_t slab = traffic >= kShortSlabBytes ? 4u : 8u;
    g.ntt = (rows + 4u * slab - 1u) / (4u * slab);
    g.L = rows;
    g.rowbytes = rowbytes;
    const uint64_t ncols = (uint64_t)batch * g.nct;
    const uint64_t grid = (ncols + 7) / 8 * 8 * g.ntt;
    if (grid >= (1ull << 31)) return 1;
    g.ncols = (uint32_t)ncols;
    if (traffic >= kThroughBytes) hipLaunchKernelGGL((copy_tiles_kernel<2 | 16, 4>), dim3((uint32_t)grid), dim3(256), 0, (hipStream_t)stream, g);
    else if (slab == 4u) hipLaunchKernelGGL((copy_tiles_kernel<2, 4>), dim3((uint32_t)grid), dim3(256), 0, (hipStream_t)stream, g);
    else hipLaunchKernelGGL((copy_tiles_kernel<2, 8>), dim3((uint32_t)grid), dim3(256), 0, (hipStream_t)stream, g);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

// shape: 0 = 32 rows x 512 B (8-byte lanes, the kernel's tile), 1 = 16 x 512 B (8-byte lanes), 2 = 16 x 1 KB and
// 3 = 32 x 1 KB (16-byte lanes), 4 = 64 x 256 B (16-byte lanes, four rows per instruction)
__attribute__((visibility("default"))) int copy_tile_shape(const void *in, void *out, uint32_t batch, uint32_t rows,
                                                           uint32_t rowbytes, int shape, void *stream)
{
    if (rowbytes % 16 || ((uintptr_t)in | (uintptr_t)out) % 16 || batch == 0 || rows == 0 || rowbytes == 0) return 1;
    if ((uint64_t)rowbytes * 40 >= (1ull << 31)) return 1;   // rows are 32-bit offsets inside a wave's resource
    hipStream_t s = (hipStream_t)stream;
    switch (shape) {
    case 0: return launch_shape<8, 8, 4, 64>(in, out, batch, rows, rowbytes, s);
    case 1: return launch_shape<8, 4, 4, 64>(in, out, batch, rows, rowbytes, s);
    case 2: return launch_shape<16, 4, 4, 64>(in, out, batch, rows, rowbytes, s);
    case 3: return launch_shape<16, 8, 4, 64>(in, out, batch, rows, rowbytes, s);
    case 4: return launch_shape<16, 4, 4, 16>(in, out, batch, rows, rowbytes, s);
    default: return 1;
    }
}

__attribute__((visibility("default"))) int empty_launch(void *stream)
{
    hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

}  // extern "C"
