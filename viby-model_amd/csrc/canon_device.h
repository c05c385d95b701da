// Device-side helpers shared by the kernels: storage-type conversions, vector
// and mask loads, tap fetch / decode, wave shifts.  Everything is
// __device__ __forceinline__ or a template, so the header may be included by
// every kernel translation unit.
#ifndef CANON_DEVICE_H
#define CANON_DEVICE_H

#include <type_traits>

#include "canon_plan.h"

namespace canon {

// ---------------------------------------------------------------------------
// storage types
// ---------------------------------------------------------------------------
template <int DT> struct Elem;
template <> struct Elem<CANON_DTYPE_F32> { static constexpr int bytes = 4; static constexpr int per_vec = 4; };
template <> struct Elem<CANON_DTYPE_BF16> { static constexpr int bytes = 2; static constexpr int per_vec = 8; };
template <> struct Elem<CANON_DTYPE_F16> { static constexpr int bytes = 2; static constexpr int per_vec = 8; };

typedef float float2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bits_f(uint32_t u) { return __uint_as_float(u); }
__device__ __forceinline__ uint32_t f_bits(float f) { return __float_as_uint(f); }

// two packed 16-bit values -> two floats
template <int DT> __device__ __forceinline__ void unpack2(uint32_t u, float &lo, float &hi)
{
    if constexpr (DT == CANON_DTYPE_BF16) {
        lo = bits_f(u << 16);
        hi = bits_f(u & 0xFFFF0000u);
    } else {
        f16x2_t h = __builtin_bit_cast(f16x2_t, u);
        lo = (float)h.x;
        hi = (float)h.y;
    }
}

// two floats -> two packed 16-bit values, round to nearest even
template <int DT> __device__ __forceinline__ uint32_t pack2(float lo, float hi)
{
    float2_t v = {lo, hi};
    if constexpr (DT == CANON_DTYPE_BF16) {
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
    } else {
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
    }
}

// value -> storage type -> value
template <int DT> __device__ __forceinline__ float round_through(float v)
{
    if constexpr (DT == CANON_DTYPE_F32) {
        return v;
    } else if constexpr (DT == CANON_DTYPE_BF16) {
        return (float)(__bf16)v;
    } else {
        return (float)(_Float16)v;
    }
}

// value -> storage type -> value where the value was just computed: for fp16 it is hidden from the
// instruction selector first, which would otherwise merge the operation that produced it and the conversion
// into one mixed-precision instruction (v_fma_mixlo_f16) whose result is not that of the two separate steps
// in every case (see mul_round below).
template <int DT> __device__ __forceinline__ float round_result(float v)
{
    if constexpr (DT == CANON_DTYPE_F16) asm volatile("" : "+v"(v));
    return round_through<DT>(v);
}

// x * m rounded to the storage type.  For fp16 the product is hidden from the
// instruction selector: it would otherwise fuse multiply and conversion into
// v_fma_mixlo_f16 with a +0 addend, which turns a -0 product into +0, and the
// captured conv state must carry the bits of x * mask exactly.
template <int DT> __device__ __forceinline__ float mul_round(float x, float m)
{
    float p = x * m;
    if constexpr (DT == CANON_DTYPE_F16) asm volatile("" : "+v"(p));
    return round_through<DT>(p);
}

template <int DT> __device__ __forceinline__ void unpack_vec(const uint4 &v, float *f)
{
    if constexpr (DT == CANON_DTYPE_F32) {
        f[0] = bits_f(v.x); f[1] = bits_f(v.y); f[2] = bits_f(v.z); f[3] = bits_f(v.w);
    } else {
        unpack2<DT>(v.x, f[0], f[1]);
        unpack2<DT>(v.y, f[2], f[3]);
        unpack2<DT>(v.z, f[4], f[5]);
        unpack2<DT>(v.w, f[6], f[7]);
    }
}

template <int DT> __device__ __forceinline__ uint4 pack_vec(const float *f)
{
    uint4 v;
    if constexpr (DT == CANON_DTYPE_F32) {
        v.x = f_bits(f[0]); v.y = f_bits(f[1]); v.z = f_bits(f[2]); v.w = f_bits(f[3]);
    } else {
        v.x = pack2<DT>(f[0], f[1]);
        v.y = pack2<DT>(f[2], f[3]);
        v.z = pack2<DT>(f[4], f[5]);
        v.w = pack2<DT>(f[6], f[7]);
    }
    return v;
}

template <int DT> __device__ __forceinline__ float load1(const void *p, int64_t i)
{
    if constexpr (DT == CANON_DTYPE_F32) {
        return ((const float *)p)[i];
    } else if constexpr (DT == CANON_DTYPE_BF16) {
        return bits_f((uint32_t)((const uint16_t *)p)[i] << 16);
    } else {
        return (float)((const _Float16 *)p)[i];
    }
}

template <int DT> __device__ __forceinline__ void store1(void *p, int64_t i, float v)
{
    if constexpr (DT == CANON_DTYPE_F32) {
        ((float *)p)[i] = v;
    } else if constexpr (DT == CANON_DTYPE_BF16) {
        ((__bf16 *)p)[i] = (__bf16)v;
    } else {
        ((_Float16 *)p)[i] = (_Float16)v;
    }
}

// weight / bias element of run-time type
__device__ __forceinline__ float load_w(const void *p, int64_t i, int dt)
{
    if (dt == CANON_DTYPE_F32) return load1<CANON_DTYPE_F32>(p, i);
    if (dt == CANON_DTYPE_BF16) return load1<CANON_DTYPE_BF16>(p, i);
    return load1<CANON_DTYPE_F16>(p, i);
}

__device__ __forceinline__ float load_mask(const void *p, int64_t i, int dt)
{
    switch (dt) {
    case CANON_MASK_U8: return (float)((const uint8_t *)p)[i];
    case CANON_MASK_I32: return (float)((const int32_t *)p)[i];
    case CANON_MASK_I64: return (float)((const int64_t *)p)[i];
    case CANON_MASK_F32: return ((const float *)p)[i];
    case CANON_MASK_BF16: return load1<CANON_DTYPE_BF16>(p, i);
    default: return load1<CANON_DTYPE_F16>(p, i);
    }
}

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

// 16-byte access; NT marks streaming data that will not be touched again soon
template <bool NT> __device__ __forceinline__ uint4 load_vec(const void *p)
{
    const u32x4_t *q = (const u32x4_t *)p;
    u32x4_t v;
    if constexpr (NT) v = __builtin_nontemporal_load(q);
    else v = *q;
    return make_uint4(v.x, v.y, v.z, v.w);
}

template <bool NT> __device__ __forceinline__ void store_vec(void *p, const uint4 &v)
{
    const u32x4_t q = {v.x, v.y, v.z, v.w};
    if constexpr (NT) __builtin_nontemporal_store(q, (u32x4_t *)p);
    else *(u32x4_t *)p = q;
}

// (float) of N 64-bit integers given as word pairs.  When every value of the whole wave fits 32 bits (the
// usual 0/1 mask) it is one conversion instruction each; otherwise the full conversions run one after the
// other.  Written as per-value selects, the N full conversions are scheduled side by side and their
// temporaries (a dozen registers each) set the register count of every kernel that can meet an int64 mask.
template <int N> __device__ __forceinline__ void i64_words_to_float_n(const uint32_t *lo, const uint32_t *hi, float *m)
{
    bool wide = false;
#pragma unroll
    for (int j = 0; j < N; ++j) wide |= (int32_t)hi[j] != ((int32_t)lo[j] >> 31);
    if (__builtin_amdgcn_ballot_w64(wide) == 0) {
#pragma unroll
        for (int j = 0; j < N; ++j) m[j] = (float)(int32_t)lo[j];
    } else {
#pragma unroll
        for (int j = 0; j < N; ++j) {
            m[j] = (float)(int64_t)(((uint64_t)hi[j] << 32) | lo[j]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// N mask entries of consecutive time steps t_first .. t_first+N-1 (clamped to
// [0, L-1]) of one batch row.  The element-type switch sits outside the loops
// and every case is straight-line code, so all N loads are issued back to back
// and waited for once (a per-entry switch puts a wait after every load, which
// also waits for -- and so serialises -- the row loads issued before it).
template <int N, bool RUN>
__device__ __forceinline__ void load_mask_entries(const void *p, int64_t first, const int64_t *idx, int dt, float *m)
{
    // RUN: the entries are first, first+1, .. (constant offsets: the loads merge); else idx[j]
    // 1- and 2-byte entries are taken out of the aligned 32-bit word that holds them: a wave-uniform
    // 32-bit load can be a scalar-memory load, a byte or short load cannot
    const uint32_t *words = (const uint32_t *)((uintptr_t)p & ~(uintptr_t)3);
    const int64_t byte0 = (int64_t)((uintptr_t)p & 3u);
    switch (dt) {
    case CANON_MASK_U8:
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const int64_t i = (RUN ? first + j : idx[j]) + byte0;
            m[j] = (float)((words[i >> 2] >> (8 * (uint32_t)(i & 3))) & 0xFFu);
        }
        break;
    case CANON_MASK_I32:
#pragma unroll
        for (int j = 0; j < N; ++j) m[j] = (float)((const int32_t *)p)[RUN ? first + j : idx[j]];
        break;
    case CANON_MASK_I64: {
        uint32_t lo[N], hi[N];
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const uint2 q = ((const uint2 *)p)[RUN ? first + j : idx[j]];
            lo[j] = q.x;
            hi[j] = q.y;
        }
        i64_words_to_float_n<N>(lo, hi, m);
        break;
    }
    case CANON_MASK_F32:
#pragma unroll
        for (int j = 0; j < N; ++j) m[j] = ((const float *)p)[RUN ? first + j : idx[j]];
        break;
    case CANON_MASK_BF16:
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const int64_t i = (RUN ? first + j : idx[j]) + (byte0 >> 1);
            const uint32_t wd = words[i >> 1];
            m[j] = bits_f((i & 1) ? (wd & 0xFFFF0000u) : (wd << 16));
        }
        break;
    default:
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const int64_t i = (RUN ? first + j : idx[j]) + (byte0 >> 1);
            const uint32_t wd = words[i >> 1];
            m[j] = (float)__builtin_bit_cast(_Float16, (uint16_t)((i & 1) ? (wd >> 16) : (wd & 0xFFFFu)));
        }
        break;
    }
}

template <int N>
__device__ __forceinline__ void load_mask_rows(const void *p, int64_t row_base, int64_t t_first, int64_t L, int64_t stride,
                                               int dt, float *m)
{
    if (stride == 1 && t_first >= 0 && t_first + N <= L) {
        // the common case, away from the ends of the sequence: one contiguous run, no clamping
        load_mask_entries<N, true>(p, row_base + t_first, nullptr, dt, m);
        return;
    }
    int64_t idx[N];
#pragma unroll
    for (int j = 0; j < N; ++j) {
        int64_t t = t_first + j;
        t = t < 0 ? 0 : (t > L - 1 ? L - 1 : t);
        idx[j] = row_base + t * stride;
    }
    load_mask_entries<N, false>(p, 0, idx, dt, m);
}

// N (<= 64) mask entries of consecutive time steps t_first .. t_first+N-1 (clamped to [0, L-1]) of one batch
// row, the same for every lane of the wave: lane j fetches entry j with one vector load, the values are then
// broadcast lane by lane.  Against one scalar load per entry this keeps eleven 64-bit addresses out of the
// scalar registers (the channel-contiguous kernel ran out of them and spilled) and puts the mask in the same
// in-order queue as the rows.
template <int N>
__device__ __forceinline__ void load_mask_rows_wave(const void *p, int64_t row_base, int64_t t_first, int64_t L,
                                                    int64_t stride, int dt, int lane, float *m)
{
    int64_t t = t_first + (lane < N ? lane : N - 1);
    t = t < 0 ? 0 : (t > L - 1 ? L - 1 : t);
    const float v = load_mask(p, row_base + t * stride, dt);
#pragma unroll
    for (int j = 0; j < N; ++j) m[j] = bits_f((uint32_t)__builtin_amdgcn_readlane((int)f_bits(v), j));
}

// The same for N sequence indices.
template <int N>
__device__ __forceinline__ void load_seq_rows_wave(const int32_t *p, int64_t row_base, int64_t t_first, int64_t L,
                                                   int64_t stride, int lane, int32_t *q)
{
    int64_t t = t_first + (lane < N ? lane : N - 1);
    t = t < 0 ? 0 : (t > L - 1 ? L - 1 : t);
    const int32_t v = p[row_base + t * stride];
#pragma unroll
    for (int j = 0; j < N; ++j) q[j] = __builtin_amdgcn_readlane(v, j);
}

// A lane's access unit in the channel-contiguous kernels: 16 bytes, or 8 bytes (half the registers
// per lane, twice the waves in flight)
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));

template <int VB> struct VecIO;
template <> struct VecIO<16> {
    using type = uint4;
    static __device__ __forceinline__ type zero() { return make_uint4(0, 0, 0, 0); }
    template <bool NT> static __device__ __forceinline__ type load(const void *p) { return load_vec<NT>(p); }
    template <bool NT> static __device__ __forceinline__ void store(void *p, const type &v) { store_vec<NT>(p, v); }
    template <int DT> static __device__ __forceinline__ void unpack(const type &v, float *f) { unpack_vec<DT>(v, f); }
    template <int DT> static __device__ __forceinline__ type pack(const float *f) { return pack_vec<DT>(f); }
};
template <> struct VecIO<8> {
    using type = uint2;
    static __device__ __forceinline__ type zero() { return make_uint2(0, 0); }
    template <bool NT> static __device__ __forceinline__ type load(const void *p)
    {
        const u32x2_t *q = (const u32x2_t *)p;
        u32x2_t v;
        if constexpr (NT) v = __builtin_nontemporal_load(q);
        else v = *q;
        return make_uint2(v.x, v.y);
    }
    template <bool NT> static __device__ __forceinline__ void store(void *p, const type &v)
    {
        const u32x2_t q = {v.x, v.y};
        if constexpr (NT) __builtin_nontemporal_store(q, (u32x2_t *)p);
        else *(u32x2_t *)p = q;
    }
    template <int DT> static __device__ __forceinline__ void unpack(const type &v, float *f)
    {
        if constexpr (DT == CANON_DTYPE_F32) {
            f[0] = bits_f(v.x);
            f[1] = bits_f(v.y);
        } else {
            unpack2<DT>(v.x, f[0], f[1]);
            unpack2<DT>(v.y, f[2], f[3]);
        }
    }
    template <int DT> static __device__ __forceinline__ type pack(const float *f)
    {
        if constexpr (DT == CANON_DTYPE_F32) return make_uint2(f_bits(f[0]), f_bits(f[1]));
        else return make_uint2(pack2<DT>(f[0], f[1]), pack2<DT>(f[2], f[3]));
    }
};

template <> struct VecIO<4> {
    using type = uint32_t;
    static __device__ __forceinline__ type zero() { return 0u; }
    template <bool NT> static __device__ __forceinline__ type load(const void *p)
    {
        const uint32_t *q = (const uint32_t *)p;
        if constexpr (NT) return __builtin_nontemporal_load(q);
        else return *q;
    }
    template <bool NT> static __device__ __forceinline__ void store(void *p, const type &v)
    {
        if constexpr (NT) __builtin_nontemporal_store(v, (uint32_t *)p);
        else *(uint32_t *)p = v;
    }
    template <int DT> static __device__ __forceinline__ void unpack(const type &v, float *f)
    {
        if constexpr (DT == CANON_DTYPE_F32) f[0] = bits_f(v);
        else unpack2<DT>(v, f[0], f[1]);
    }
    template <int DT> static __device__ __forceinline__ type pack(const float *f)
    {
        if constexpr (DT == CANON_DTYPE_F32) return f_bits(f[0]);
        else return pack2<DT>(f[0], f[1]);
    }
};

// Buffer accesses: address = resource base + vector offset + scalar offset, the sum checked against the
// resource's size (measured on this hardware: the scalar offset counts; an access beyond the size loads zeros
// and stores nothing).  A resource therefore spans every row its wave touches, and lanes that must not access
// memory get a vector offset beyond any size.
constexpr int kBufFlags = 0x00020000;   // raw buffer, 32-bit data format
// Cache policy of a buffer access (its auxiliary bits).  Streamed data (x is read once, out written once) is
// marked non-temporal whatever its size: measured on plain copies of 10 .. 450 MB each way, 9-17 % faster than
// default accesses.  The channel-contiguous prefill marks the stores of a large launch system scope as well
// (written through: the end of the kernel has no dirty L2 lines left to write back): 0.4 us of 21 us at B = 8,
// 0.7 of 74 us at B = 32.  A plain copy of 10 MB each way loses 0.4 us to the same bit, hence the size
// threshold, and the time-contiguous kernel (1 KB per store instruction and wave) loses 0.1 .. 0.8 us, so it
// does not use it.
constexpr int kAuxPlain = 0, kAuxStream = 2 /* nt */, kAuxStreamThrough = 2 | 16 /* nt sc1 */;
template <bool BIG> constexpr int store_policy() { return BIG ? kAuxStreamThrough : kAuxStream; }

template <int VB> struct BufIO;
template <> struct BufIO<8> {
    template <int AUX> static __device__ __forceinline__ uint2 load(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff)
    {
        const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(r, (int)voff, (int)soff, AUX);
        return make_uint2(v.x, v.y);
    }
    template <int AUX> static __device__ __forceinline__ void store(const uint2 &v, __amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff)
    {
        const u32x2_t q = {v.x, v.y};
        __builtin_amdgcn_raw_buffer_store_b64(q, r, (int)voff, (int)soff, AUX);
    }
};
template <> struct BufIO<16> {
    template <int AUX> static __device__ __forceinline__ uint4 load(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff)
    {
        const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, AUX);
        return make_uint4(v.x, v.y, v.z, v.w);
    }
    template <int AUX> static __device__ __forceinline__ void store(const uint4 &v, __amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff)
    {
        const u32x4_t q = {v.x, v.y, v.z, v.w};
        __builtin_amdgcn_raw_buffer_store_b128(q, r, (int)voff, (int)soff, AUX);
    }
};

// N consecutive 32-bit words through a buffer resource (zeros where out of its range)
template <int N> __device__ __forceinline__ void buf_load_words(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t *d)
{
    if constexpr (N == 1) {
        d[0] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(r, (int)voff, 0, 0);
    } else if constexpr (N == 2) {
        const u32x2_t q = __builtin_amdgcn_raw_buffer_load_b64(r, (int)voff, 0, 0);
        d[0] = q.x; d[1] = q.y;
    } else if constexpr (N == 4) {
        const u32x4_t q = __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, 0, 0);
        d[0] = q.x; d[1] = q.y; d[2] = q.z; d[3] = q.w;
    } else {
        static_assert(N % 4 == 0 && N > 4, "1, 2 or a multiple of 4 words");
        buf_load_words<4>(r, voff, d);
        buf_load_words<N - 4>(r, voff + 16u, d + 4);
    }
}

// N sequence indices of consecutive time steps t_first .. t_first+N-1 (clamped to [0, L-1]) of one batch row
template <int N>
__device__ __forceinline__ void load_seq_rows(const int32_t *p, int64_t row_base, int64_t t_first, int64_t L, int64_t stride,
                                              int32_t *q)
{
#pragma unroll
    for (int j = 0; j < N; ++j) {
        int64_t t = t_first + j;
        t = t < 0 ? 0 : (t > L - 1 ? L - 1 : t);
        q[j] = p[row_base + t * stride];
    }
}

// U runs of N (4 or 8) consecutive mask entries, run u starting at element
// base[u].  The element-type switch sits outside the loops and every case is
// straight-line code, so all loads are issued back to back and waited for
// once.  `vec` (decided on the host) says the entries are contiguous and each
// run is aligned to its own size: it is fetched with a few wide loads instead
// of N narrow ones.
template <int N, int U>
__device__ __forceinline__ void load_mask_vec(const void *p, const int64_t *base, int64_t stride, int dt, bool vec,
                                              float (*m)[N])
{
    if (vec) {
        switch (dt) {
        case CANON_MASK_U8: {
            uint32_t q[U][N / 4];
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int i = 0; i < N / 4; ++i) q[u][i] = ((const uint32_t *)((const uint8_t *)p + base[u]))[i];
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int j = 0; j < N; ++j) m[u][j] = (float)((q[u][j / 4] >> (8 * (j % 4))) & 0xFFu);
            return;
        }
        case CANON_MASK_I32: {
#pragma unroll
            for (int u = 0; u < U; ++u) {   // one vector at a time, as for int64 below
                uint4 q[N / 4 > 0 ? N / 4 : 1];   // (N < 4 never takes the vector path)
#pragma unroll
                for (int i = 0; i < N / 4; ++i) q[i] = ((const uint4 *)((const int32_t *)p + base[u]))[i];
#pragma unroll
                for (int i = 0; i < N / 4; ++i) {
                    m[u][4 * i] = (float)(int32_t)q[i].x; m[u][4 * i + 1] = (float)(int32_t)q[i].y;
                    m[u][4 * i + 2] = (float)(int32_t)q[i].z; m[u][4 * i + 3] = (float)(int32_t)q[i].w;
                }
                if (u + 1 < U) __builtin_amdgcn_sched_barrier(0);
            }
            return;
        }
        case CANON_MASK_I64: {
            // one vector's entries (N / 2 16-byte loads) at a time: holding the raw words of all U vectors would
            // set the register count of the whole kernel (all mask types share it) and cost a wave per SIMD
#pragma unroll
            for (int u = 0; u < U; ++u) {
                uint4 q[N / 2 > 0 ? N / 2 : 1];
#pragma unroll
                for (int i = 0; i < N / 2; ++i) q[i] = ((const uint4 *)((const int64_t *)p + base[u]))[i];
                uint32_t lo[N], hi[N];
#pragma unroll
                for (int i = 0; i < N / 2; ++i) {
                    lo[2 * i] = q[i].x; hi[2 * i] = q[i].y;
                    lo[2 * i + 1] = q[i].z; hi[2 * i + 1] = q[i].w;
                }
                i64_words_to_float_n<N>(lo, hi, m[u]);
                if (u + 1 < U) __builtin_amdgcn_sched_barrier(0);   // keep the next vector's loads behind this conversion
            }
            return;
        }
        case CANON_MASK_F32: {
            uint4 q[U][N / 4];
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int i = 0; i < N / 4; ++i) q[u][i] = ((const uint4 *)((const float *)p + base[u]))[i];
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int i = 0; i < N / 4; ++i) {
                    m[u][4 * i] = bits_f(q[u][i].x); m[u][4 * i + 1] = bits_f(q[u][i].y);
                    m[u][4 * i + 2] = bits_f(q[u][i].z); m[u][4 * i + 3] = bits_f(q[u][i].w);
                }
            return;
        }
        default: {   // bf16 / fp16
            uint32_t q[U][N / 2];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if constexpr (N == 8) {
                    const uint4 v = *(const uint4 *)((const uint16_t *)p + base[u]);
                    q[u][0] = v.x; q[u][1] = v.y; q[u][2 % (N / 2)] = v.z; q[u][3 % (N / 2)] = v.w;
                } else {
                    const uint2 v = *(const uint2 *)((const uint16_t *)p + base[u]);
                    q[u][0] = v.x; q[u][1] = v.y;
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int i = 0; i < N / 2; ++i) {
                    if (dt == CANON_MASK_BF16) unpack2<CANON_DTYPE_BF16>(q[u][i], m[u][2 * i], m[u][2 * i + 1]);
                    else unpack2<CANON_DTYPE_F16>(q[u][i], m[u][2 * i], m[u][2 * i + 1]);
                }
            return;
        }
        }
    }
    switch (dt) {
    case CANON_MASK_U8:
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < N; ++j) m[u][j] = (float)((const uint8_t *)p)[base[u] + j * stride];
        break;
    case CANON_MASK_I32:
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < N; ++j) m[u][j] = (float)((const int32_t *)p)[base[u] + j * stride];
        break;
    case CANON_MASK_I64:
#pragma unroll
        for (int u = 0; u < U; ++u) {
            uint32_t lo[N], hi[N];
#pragma unroll
            for (int j = 0; j < N; ++j) {
                const uint2 q = ((const uint2 *)p)[base[u] + j * stride];
                lo[j] = q.x;
                hi[j] = q.y;
            }
            i64_words_to_float_n<N>(lo, hi, m[u]);
        }
        break;
    case CANON_MASK_F32:
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < N; ++j) m[u][j] = ((const float *)p)[base[u] + j * stride];
        break;
    case CANON_MASK_BF16:
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < N; ++j) m[u][j] = load1<CANON_DTYPE_BF16>(p, base[u] + j * stride);
        break;
    default:
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < N; ++j) m[u][j] = load1<CANON_DTYPE_F16>(p, base[u] + j * stride);
        break;
    }
}

__device__ __forceinline__ float silu_fast(float v)
{
    // v / (1 + e^-v); v_exp_f32 and v_rcp_f32 are each good to 1 ulp
    return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v));
}

__device__ __forceinline__ float silu_precise(float v) { return v / (1.0f + expf(-v)); }

// lane i <- lane i-1 across the whole wave; lane 0 <- `first`
__device__ __forceinline__ float wave_shift_up(float v, float first)
{
    return bits_f((uint32_t)__builtin_amdgcn_update_dpp((int)f_bits(first), (int)f_bits(v),
                                                        0x138 /* wave_shr:1 */, 0xF, 0xF, false));
}

__device__ __forceinline__ float read_lane63(float v)
{
    return bits_f((uint32_t)__builtin_amdgcn_readlane((int)f_bits(v), 63));
}

__device__ __forceinline__ uint32_t fdiv(uint32_t n, const FastDiv &f)
{
    const uint32_t t = __umulhi(f.m, n);
    return (t + ((n - t) >> f.s1)) >> f.s2;
}

// Activation of N accumulators.  Fused rounding: fp32 throughout (the only rounding is the one at the
// store).  Eager rounding: the eager module's rounding points, i.e. the convolution result is rounded to the
// storage type, and so is the activation (the residual sum is rounded by the store).
template <int DT, int N> __device__ __forceinline__ void activate(float *o, bool act, bool eager)
{
    if (eager) {
#pragma unroll
        for (int j = 0; j < N; ++j) o[j] = round_result<DT>(o[j]);
        if (act) {
#pragma unroll
            for (int j = 0; j < N; ++j) o[j] = round_result<DT>(silu_precise(o[j]));
        }
    } else if (act) {
#pragma unroll
        for (int j = 0; j < N; ++j) o[j] = silu_fast(o[j]);
    }
}

// The activated, residual-added output of one element.
template <int DT> __device__ __forceinline__ float finish(float acc, int act, int res_mode, int eager, float xm, float xr)
{
    activate<DT, 1>(&acc, act != 0, eager != 0);
    if (res_mode == CANON_RESIDUAL_MASKED) acc += xm;
    else if (res_mode == CANON_RESIDUAL_UNMASKED) acc += xr;
    return acc;
}

// Write final_state[b, c, :] for one row from global memory (the row was just
// streamed by this wave, so these are cache hits).  One lane per slot.
template <int DT>
__device__ __forceinline__ void capture_row_state(const FwdArgs &a, uint32_t b, uint32_t c, int slot)
{
    if (slot >= a.S_out) return;
    const int64_t t = (int64_t)a.L - a.S_out + slot;
    float v = 0.0f;
    if (t >= 0) {
        v = load1<DT>(a.x, b * a.x_sb + c * a.x_sc + t * a.x_sl);
        if (a.mask) v = mul_round<DT>(v, load_mask(a.mask, b * a.m_sb + t * a.m_sl, a.mask_dtype));
    } else if (a.init && a.S_in + t >= 0) {
        v = load1<DT>(a.init, b * a.i_sb + c * a.i_sc + (a.S_in + t) * a.i_ss);
    }
    store1<DT>(a.fin, b * a.f_sb + c * a.f_sc + slot * a.f_ss, v);
}

// Taps and bias of NC adjacent channels, in two phases so that the loads can
// be issued early and nothing waits on them until the values are needed:
// fetch_taps() only loads raw bits, decode_taps() converts them (rounded to
// the storage type of x).  `vec` (decided on the host): weight is a
// contiguous, 16-byte aligned [C, 4].
template <int NC> struct RawTaps {
    uint32_t w[NC][4];   // fp32: one tap per word; 16-bit + vec: two taps per word in w[.][0..1];
                         // 16-bit scalar path: one tap per word, low half
    uint32_t b[NC];
};

template <int W, int NC>
__device__ __forceinline__ void fetch_taps(const void *weight, const void *bias, int64_t w_sc, int64_t w_sk,
                                           int w_dtype, bool vec, uint32_t c0, RawTaps<NC> &r)
{
    const bool wide = w_dtype == CANON_DTYPE_F32;
    // bias first: whatever follows the tap loads may wait on them, and nothing must be issued after a wait
    if (bias) {
        if (wide) {
#pragma unroll
            for (int e = 0; e < NC; ++e) r.b[e] = ((const uint32_t *)bias)[c0 + e];
        } else {
#pragma unroll
            for (int e = 0; e < NC; ++e) r.b[e] = ((const uint16_t *)bias)[c0 + e];
        }
    }
    if (W == 4 && vec) {
        if (wide) {
            const uint4 *p = (const uint4 *)weight + c0;
#pragma unroll
            for (int e = 0; e < NC; ++e) {
                const uint4 q = p[e];
                r.w[e][0] = q.x; r.w[e][1] = q.y; r.w[e][2] = q.z; r.w[e][3] = q.w;
            }
        } else if constexpr (NC % 2 == 0) {
            const uint4 *p = (const uint4 *)((const uint2 *)weight + c0);   // c0 is a multiple of NC
#pragma unroll
            for (int e = 0; e < NC; e += 2) {
                const uint4 q = p[e / 2];
                r.w[e][0] = q.x; r.w[e][1] = q.y;
                r.w[e + 1][0] = q.z; r.w[e + 1][1] = q.w;
            }
        } else {
            const uint2 *p = (const uint2 *)weight + c0;
#pragma unroll
            for (int e = 0; e < NC; ++e) {
                const uint2 q = p[e];
                r.w[e][0] = q.x; r.w[e][1] = q.y;
            }
        }
    } else if (wide) {
#pragma unroll
        for (int e = 0; e < NC; ++e)
#pragma unroll
            for (int k = 0; k < W; ++k) r.w[e][k] = ((const uint32_t *)weight)[(int64_t)(c0 + e) * w_sc + k * w_sk];
    } else {
#pragma unroll
        for (int e = 0; e < NC; ++e)
#pragma unroll
            for (int k = 0; k < W; ++k) r.w[e][k] = ((const uint16_t *)weight)[(int64_t)(c0 + e) * w_sc + k * w_sk];
    }
}

// One channel's taps for a whole wave (c is wave-uniform): shaped so that the
// common cases become scalar-memory loads.  `pair`: bias may be read as the
// aligned 32-bit word that contains element c.
template <int W>
__device__ __forceinline__ void fetch_taps_uniform(const void *weight, const void *bias, int64_t w_sc, int64_t w_sk,
                                                   int w_dtype, bool vec, bool pair, uint32_t c, RawTaps<1> &r)
{
    const bool wide = w_dtype == CANON_DTYPE_F32;
    if (bias && pair) {
        if (wide) {
            r.b[0] = ((const uint32_t *)bias)[c];
        } else {
            const uint32_t d = ((const uint32_t *)bias)[c >> 1];
            r.b[0] = (c & 1u) ? (d >> 16) : (d & 0xFFFFu);
        }
        fetch_taps<W, 1>(weight, nullptr, w_sc, w_sk, w_dtype, vec, c, r);
    } else {
        fetch_taps<W, 1>(weight, bias, w_sc, w_sk, w_dtype, vec, c, r);
    }
}

template <int WDT> __device__ __forceinline__ float half_bits_f(uint32_t raw)
{
    if constexpr (WDT == CANON_DTYPE_BF16) return bits_f(raw << 16);
    else return (float)__builtin_bit_cast(_Float16, (uint16_t)raw);
}

template <int DT, int WDT, int W, int NC>
__device__ __forceinline__ void decode_taps_typed(const RawTaps<NC> &r, bool vec, bool has_bias, float (*w)[W], float *bv)
{
#pragma unroll
    for (int e = 0; e < NC; ++e) {
        if constexpr (WDT == CANON_DTYPE_F32) {
#pragma unroll
            for (int k = 0; k < W; ++k) w[e][k] = round_through<DT>(bits_f(r.w[e][k]));
            bv[e] = has_bias ? round_through<DT>(bits_f(r.b[e])) : 0.0f;
        } else {
            if (W == 4 && vec) {
                float t0, t1, t2, t3;
                unpack2<WDT>(r.w[e][0], t0, t1);
                unpack2<WDT>(r.w[e][1], t2, t3);
                w[e][0] = round_through<DT>(t0);
                w[e][1] = round_through<DT>(t1);
                w[e][W - 2] = round_through<DT>(t2);
                w[e][W - 1] = round_through<DT>(t3);
            } else {
#pragma unroll
                for (int k = 0; k < W; ++k) w[e][k] = round_through<DT>(half_bits_f<WDT>(r.w[e][k]));
            }
            bv[e] = has_bias ? round_through<DT>(half_bits_f<WDT>(r.b[e])) : 0.0f;
        }
    }
}

template <int DT, int W, int NC>
__device__ __forceinline__ void decode_taps(const RawTaps<NC> &r, int w_dtype, bool vec, bool has_bias, float (*w)[W], float *bv)
{
    // weights that already have the storage type of x need no rounding: decode them as if x were fp32
    if (w_dtype == DT) decode_taps_typed<CANON_DTYPE_F32, DT, W, NC>(r, vec, has_bias, w, bv);
    else if (w_dtype == CANON_DTYPE_F32) decode_taps_typed<DT, CANON_DTYPE_F32, W, NC>(r, vec, has_bias, w, bv);
    else if (w_dtype == CANON_DTYPE_BF16) decode_taps_typed<DT, CANON_DTYPE_BF16, W, NC>(r, vec, has_bias, w, bv);
    else decode_taps_typed<DT, CANON_DTYPE_F16, W, NC>(r, vec, has_bias, w, bv);
}

// ---------------------------------------------------------------------------
// Runs of 32-bit words at 4-byte aligned addresses, and elements of a storage
// type packed in such words (raw bits)
// ---------------------------------------------------------------------------
typedef uint32_t words2_t __attribute__((ext_vector_type(2), aligned(4)));
typedef uint32_t words3_t __attribute__((ext_vector_type(3), aligned(4)));
typedef uint32_t words4_t __attribute__((ext_vector_type(4), aligned(4)));

// N consecutive 32-bit words at a 4-byte aligned address
template <int N> __device__ __forceinline__ void load_words(const char *p, uint32_t *d)
{
    if constexpr (N == 1) {
        d[0] = *(const uint32_t *)p;
    } else if constexpr (N == 2) {
        const words2_t q = *(const words2_t *)p;
        d[0] = q.x; d[1] = q.y;
    } else if constexpr (N == 3) {
        const words3_t q = *(const words3_t *)p;
        d[0] = q.x; d[1] = q.y; d[2] = q.z;
    } else if constexpr (N == 4) {
        const words4_t q = *(const words4_t *)p;
        d[0] = q.x; d[1] = q.y; d[2] = q.z; d[3] = q.w;
    } else {
        load_words<4>(p, d);
        load_words<N - 4>(p + 16, d + 4);
    }
}

template <int N> __device__ __forceinline__ void store_words(char *p, const uint32_t *d)
{
    if constexpr (N == 1) {
        *(uint32_t *)p = d[0];
    } else if constexpr (N == 2) {
        words2_t q; q.x = d[0]; q.y = d[1];
        *(words2_t *)p = q;
    } else if constexpr (N == 3) {
        words3_t q; q.x = d[0]; q.y = d[1]; q.z = d[2];
        *(words3_t *)p = q;
    } else if constexpr (N == 4) {
        words4_t q; q.x = d[0]; q.y = d[1]; q.z = d[2]; q.w = d[3];
        *(words4_t *)p = q;
    } else {
        store_words<4>(p, d);
        store_words<N - 4>(p + 16, d + 4);
    }
}

// elements of the storage type packed in 32-bit words, handled as raw bits
template <int DT> struct Packed {
    static __device__ __forceinline__ uint32_t get(const uint32_t *d, int i)
    {
        if constexpr (DT == CANON_DTYPE_F32) return d[i];
        else return (i & 1) ? (d[i >> 1] >> 16) : (d[i >> 1] & 0xFFFFu);
    }
    static __device__ __forceinline__ void put(uint32_t *d, int i, uint32_t raw)   // d starts as zeros
    {
        if constexpr (DT == CANON_DTYPE_F32) d[i] = raw;
        else d[i >> 1] |= (i & 1) ? (raw << 16) : raw;
    }
    static __device__ __forceinline__ float as_float(uint32_t raw)
    {
        if constexpr (DT == CANON_DTYPE_F32) return bits_f(raw);
        else if constexpr (DT == CANON_DTYPE_BF16) return bits_f(raw << 16);
        else return (float)__builtin_bit_cast(_Float16, (uint16_t)raw);
    }
    static __device__ __forceinline__ uint32_t raw_of(float f)   // rounds to nearest even
    {
        if constexpr (DT == CANON_DTYPE_F32) return f_bits(f);
        else if constexpr (DT == CANON_DTYPE_BF16) return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f);
        else return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
    }
};

// Taps and bias of E adjacent channels from a contiguous [C, 4] weight array of
// type WDT (16-byte aligned; bias 4-byte aligned): straight-line loads, no
// branch on a run-time type between them, so a kernel can have them in flight
// together with everything else it requests.
template <int WDT, int E> struct TapWords {
    static constexpr int NW = E * Elem<WDT>::bytes;               // 4 taps per channel
    static constexpr int NB = (E * Elem<WDT>::bytes + 3) / 4;
    uint32_t w[NW];
    uint32_t b[NB];
};

template <int WDT, int E>
__device__ __forceinline__ void fetch_taps_contiguous(const void *weight, const void *bias, uint32_t c0, TapWords<WDT, E> &r)
{
    constexpr int WBY = Elem<WDT>::bytes;
    load_words<TapWords<WDT, E>::NW>((const char *)weight + (int64_t)c0 * 4 * WBY, r.w);
    // no branch around the bias load (a merge of "loaded" and "zero" costs a wait): without a bias the same
    // bytes are read from the weights, which are at least as long, and ignored when decoding
    const char *bp = (const char *)(bias ? bias : weight) + (int64_t)c0 * WBY;
    if constexpr (E * WBY == 2) r.b[0] = *(const uint16_t *)bp;
    else load_words<TapWords<WDT, E>::NB>(bp, r.b);
}

// ... converted to float and rounded to the storage type DT of x (zero bias when there is none)
template <int DT, int WDT, int E>
__device__ __forceinline__ void decode_taps_contiguous(const TapWords<WDT, E> &r, bool has_bias, float (*w)[4], float *bv)
{
#pragma unroll
    for (int e = 0; e < E; ++e) {
#pragma unroll
        // weights that already have the storage type of x need no rounding
        for (int k = 0; k < 4; ++k) {
            const float t = Packed<WDT>::as_float(Packed<WDT>::get(r.w, e * 4 + k));
            w[e][k] = WDT == DT ? t : round_through<DT>(t);
        }
        const float tb = Packed<WDT>::as_float(Packed<WDT>::get(r.b, e));
        bv[e] = has_bias ? (WDT == DT ? tb : round_through<DT>(tb)) : 0.0f;
    }
}

// Where a block gets its argument block from.  ArgsRead: it was read at the start of the kernel (what every
// kernel does when the library is built with -DCANON_NO_LATE_ARGS).  ArgsToRead: it
// is read from the kernel-argument segment AFTER the block has requested its data from the kernel's leading
// scalar arguments, which arrive in registers with the wave (kernel-argument preload): the data loads are on
// their way while the argument block is read.  The empty asm is what orders the two: it may write memory, so
// the data loads stay in front of it, and the argument pointer comes out of it, so the argument loads stay
// behind it (left alone the compiler hoists them to the top of the kernel and waits for them there).
template <typename A> struct ArgsRead {
    static constexpr bool kLate = false;
    const A &a;
    __device__ __forceinline__ const A &get() const { return a; }
};
template <typename A> struct ArgsToRead {
    static constexpr bool kLate = true;
    uint32_t offset;   // of the argument block in the kernel-argument segment
    __device__ __forceinline__ A get() const
    {
        typedef __attribute__((address_space(4))) const char *kernarg_ptr;
        kernarg_ptr p = (kernarg_ptr)__builtin_amdgcn_kernarg_segment_ptr() + offset;
        asm volatile("" : "+s"(p) : : "memory");
        typedef __attribute__((address_space(4))) const A *args_ptr;   // (aligned: scalar loads)
        A a;
        __builtin_memcpy(&a, (args_ptr)p, sizeof(A));
        return a;
    }
};

// A kernel's leading scalar arguments are listed once, as X(type, name) entries of a macro, and expanded with these
// two into its signature and into the struct that mirrors its kernel-argument segment: the offset of the argument
// block that follows them cannot drift from the signature.
#define CANON_LEAD_PARAM(type, name) type name,
#define CANON_LEAD_FIELD(type, name) type name;

template <typename Args>
__device__ __forceinline__ uint32_t part_of_block(const PartTable<Args> &m, uint32_t blk)
{
    uint32_t p = 0;
#pragma unroll
    for (int i = 1; i < kMaxParts; ++i) p += blk >= m.first_block[i] ? 1u : 0u;
    return p;
}

}  // namespace canon
#endif  // CANON_DEVICE_H
