// Canon causal depthwise conv1d for MI355X (gfx950, wave64): prefill and
// single-token decode update, behind the C ABI of include/canon_conv1d.h.
//
// The op is a width-<=4 FIR per (batch, channel) row: ~2 flop per byte moved,
// so every kernel here is organised around HBM traffic, not arithmetic:
//   * one 16-byte load and one 16-byte store per lane per vector, each element
//     of x read from HBM once and each element of out written once;
//   * the (W-1)-element history a vector needs comes from the neighbouring
//     lane (DPP wave shift) or from the previous vector of the same wave held
//     in registers; only the first lane of a row segment touches memory for it;
//   * taps and bias live in registers; bias, SiLU, mask multiply, residual and
//     the conv-state capture are fused into the same pass.
//
// Arithmetic contract (the tests hold a CPU restatement of exactly this):
//     acc = bias;  for k in 0..W-1: acc = fmaf(w[k], xm[t-(W-1)+k], acc)
// taps/bias rounded to the storage type of x first; one rounding at the store.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdlib.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include <type_traits>

#include "canon_conv1d.h"

// build-time tuning knobs of the channel-contiguous prefill kernel
#ifndef CANON_BLC_ROWS
#define CANON_BLC_ROWS 8
#endif

namespace {

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

// (float) of a 64-bit integer given as two words; masks are 0/1 in practice, so
// the value almost always fits 32 bits and one conversion instruction does it
__device__ __forceinline__ float i64_words_to_float(uint32_t lo, uint32_t hi)
{
    if ((int32_t)hi == ((int32_t)lo >> 31)) return (float)(int32_t)lo;
    return (float)(int64_t)(((uint64_t)hi << 32) | lo);
}

// N mask entries of consecutive time steps t_first .. t_first+N-1 (clamped to
// [0, L-1]) of one batch row.  The element-type switch sits outside the loops
// and every case is straight-line code, so all N loads are issued back to back
// and waited for once (a per-entry switch puts a wait after every load, which
// also waits for -- and so serialises -- the row loads issued before it).
template <int N>
__device__ __forceinline__ void load_mask_rows(const void *p, int64_t row_base, int64_t t_first, int64_t L, int64_t stride,
                                               int dt, float *m)
{
    int64_t idx[N];
#pragma unroll
    for (int j = 0; j < N; ++j) {
        int64_t t = t_first + j;
        t = t < 0 ? 0 : (t > L - 1 ? L - 1 : t);
        idx[j] = row_base + t * stride;
    }
    switch (dt) {
    case CANON_MASK_U8:
#pragma unroll
        for (int j = 0; j < N; ++j) m[j] = (float)((const uint8_t *)p)[idx[j]];
        break;
    case CANON_MASK_I32:
#pragma unroll
        for (int j = 0; j < N; ++j) m[j] = (float)((const int32_t *)p)[idx[j]];
        break;
    case CANON_MASK_I64: {
        uint2 q[N];
#pragma unroll
        for (int j = 0; j < N; ++j) q[j] = ((const uint2 *)p)[idx[j]];
#pragma unroll
        for (int j = 0; j < N; ++j) m[j] = i64_words_to_float(q[j].x, q[j].y);
        break;
    }
    case CANON_MASK_F32:
#pragma unroll
        for (int j = 0; j < N; ++j) m[j] = ((const float *)p)[idx[j]];
        break;
    case CANON_MASK_BF16:
#pragma unroll
        for (int j = 0; j < N; ++j) m[j] = load1<CANON_DTYPE_BF16>(p, idx[j]);
        break;
    default:
#pragma unroll
        for (int j = 0; j < N; ++j) m[j] = load1<CANON_DTYPE_F16>(p, idx[j]);
        break;
    }
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
            uint4 q[U][N / 4];
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int i = 0; i < N / 4; ++i) q[u][i] = ((const uint4 *)((const int32_t *)p + base[u]))[i];
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int i = 0; i < N / 4; ++i) {
                    m[u][4 * i] = (float)(int32_t)q[u][i].x; m[u][4 * i + 1] = (float)(int32_t)q[u][i].y;
                    m[u][4 * i + 2] = (float)(int32_t)q[u][i].z; m[u][4 * i + 3] = (float)(int32_t)q[u][i].w;
                }
            return;
        }
        case CANON_MASK_I64: {
            uint4 q[U][N / 2];
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int i = 0; i < N / 2; ++i) q[u][i] = ((const uint4 *)((const int64_t *)p + base[u]))[i];
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int i = 0; i < N / 2; ++i) {
                    m[u][2 * i] = i64_words_to_float(q[u][i].x, q[u][i].y);
                    m[u][2 * i + 1] = i64_words_to_float(q[u][i].z, q[u][i].w);
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
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < N; ++j) m[u][j] = (float)((const int64_t *)p)[base[u] + j * stride];
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

// Division by a run-time constant as multiply-high and shifts (set up on the host).
struct FastDiv {
    uint32_t d, m, s1, s2;
};

__device__ __forceinline__ uint32_t fdiv(uint32_t n, const FastDiv &f)
{
    const uint32_t t = __umulhi(f.m, n);
    return (t + ((n - t) >> f.s1)) >> f.s2;
}

// ---------------------------------------------------------------------------
// kernel argument blocks (device copies of the validated ABI structs)
// ---------------------------------------------------------------------------
struct FwdArgs {
    const char *x;
    char *out;
    const void *weight;
    const void *bias;
    const void *mask;
    const void *init;
    void *fin;
    const int32_t *seq;
    int64_t q_sb, q_sl;
    int64_t x_sb, x_sc, x_sl;
    int64_t o_sb, o_sc, o_sl;
    int64_t w_sc, w_sk;
    int64_t m_sb, m_sl;
    int64_t i_sb, i_sc, i_ss;
    int64_t f_sb, f_sc, f_ss;
    uint32_t B, C, L;
    int32_t W, w_dtype, mask_dtype, act, res_mode, eager, S_in, S_out, w_vec, b_vec, b_pair, m_vec, nt;
    // launch geometry
    uint32_t nvec;      // bcl: vectors per row        blc: channel vectors per time row
    uint32_t nseg;      // bcl: segments per row       generic: time chunks per row
    uint32_t chunk;     // generic: time steps per chunk
    uint32_t ntasks;    // bcl: wave tasks   blc: blocks   generic: threads
    uint32_t nblocks;   // blocks to launch
    FastDiv div_nseg, div_C;
    // blc: tiles
    uint32_t nct, ntt;  // channel tiles per row, time tiles per sequence
    FastDiv div_nct, div_ntt;
};

struct UpdArgs {
    const char *x;
    char *out;
    char *state;
    const void *weight;
    const void *bias;
    const void *tmask;
    int64_t x_sb, x_sc, o_sb, o_sc;
    int64_t s_sb, s_sc, s_ss;
    int64_t w_sc, w_sk;
    int64_t m_sb;
    uint32_t B, C;
    int32_t W, S, w_dtype, mask_dtype, act, res_mode, eager, w_vec, b_vec;
    uint32_t nvec;      // channel vectors per batch row
    uint32_t bgroups;   // batch groups (each thread walks nb batch rows)
    uint32_t nb;
    uint32_t nthreads;
    FastDiv div_nvec;
};

// The activated, residual-added output of one element (fused rounding mode).
__device__ __forceinline__ float finish(float acc, int act, int res_mode, float xm, float xr)
{
    if (act) acc = silu_fast(acc);
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
                                           int w_dtype, bool vec, bool bvec, uint32_t c0, RawTaps<NC> &r)
{
    const bool wide = w_dtype == CANON_DTYPE_F32;
    // bias first: whatever follows the tap loads may wait on them, and nothing must be issued after a wait
    if (bias) {
        if (wide) {
#pragma unroll
            for (int e = 0; e < NC; ++e) r.b[e] = ((const uint32_t *)bias)[c0 + e];
        } else if (NC == 8 && bvec) {
            // eight 16-bit biases are one aligned 16-byte run (c0 is a multiple of 8)
            const uint4 q = *(const uint4 *)((const uint16_t *)bias + c0);
            r.b[0] = q.x & 0xFFFFu; r.b[1 % NC] = q.x >> 16;
            r.b[2 % NC] = q.y & 0xFFFFu; r.b[3 % NC] = q.y >> 16;
            r.b[4 % NC] = q.z & 0xFFFFu; r.b[5 % NC] = q.z >> 16;
            r.b[6 % NC] = q.w & 0xFFFFu; r.b[7 % NC] = q.w >> 16;
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
        fetch_taps<W, 1>(weight, nullptr, w_sc, w_sk, w_dtype, vec, false, c, r);
    } else {
        fetch_taps<W, 1>(weight, bias, w_sc, w_sk, w_dtype, vec, false, c, r);
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
// prefill, time-contiguous rows ([B, C, L], x_stride_l == 1)
//
// One wave owns one segment of one (b, c) row: U vectors per lane, lane l of
// step u holding elements [(seg*U + u)*64 + l] * E .. +E.  All U loads are
// issued before any arithmetic.  The three elements before a vector come from
// lane l-1 (wave shift), for lane 0 from lane 63 of the previous step, and for
// the very first vector of the segment from memory / the initial state / zero.
// Everything that does not change per element (activation, residual, mask
// element type) is branched on once per vector, never per element, so the
// unmasked path is ~130 VALU instructions per 2 KB row and hides under the
// memory time.
// ---------------------------------------------------------------------------
template <int DT, int W, int U, bool MASK, bool NT>
__global__ __launch_bounds__(256) void canon_fwd_bcl_kernel(const FwdArgs a)
{
    constexpr int E = Elem<DT>::per_vec;
    const int lane = threadIdx.x & 63;
    const uint32_t task = __builtin_amdgcn_readfirstlane(blockIdx.x * 4u + (threadIdx.x >> 6));
    if (task >= a.ntasks) return;
    uint32_t row = task, seg = 0;
    if (a.nseg > 1) {
        row = fdiv(task, a.div_nseg);
        seg = task - row * a.nseg;
    }
    const uint32_t b = fdiv(row, a.div_C);
    const uint32_t c = row - b * a.C;

    const char *xrow = a.x + ((int64_t)b * a.x_sb + (int64_t)c * a.x_sc) * Elem<DT>::bytes;
    char *orow = a.out + ((int64_t)b * a.o_sb + (int64_t)c * a.o_sc) * Elem<DT>::bytes;
    const uint32_t v0 = seg * (64u * U) + lane;

    // row data first (the long latency), then the taps (scalar-cache hits)
    uint4 X[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t v = v0 + u * 64u;
        X[u] = make_uint4(0, 0, 0, 0);
        if (v < a.nvec) X[u] = load_vec<NT>(xrow + (int64_t)v * 16);
    }

    RawTaps<1> raw;
    fetch_taps_uniform<W>(a.weight, a.bias, a.w_sc, a.w_sk, a.w_dtype, a.w_vec != 0, a.b_pair != 0, c, raw);

    // all mask entries of the segment, requested before anything is consumed
    float M[MASK ? U : 1][E];
    if constexpr (MASK) {
        int64_t mbase[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t v = v0 + u * 64u;
            mbase[u] = b * a.m_sb + (int64_t)(v < a.nvec ? v : a.nvec - 1u) * E * a.m_sl;   // idle lanes shadow the last vector
        }
        load_mask_vec<E, U>(a.mask, mbase, a.m_sl, a.mask_dtype, a.m_vec != 0, M);
    }

    float w[1][W], bvv[1];
    decode_taps<DT, W, 1>(raw, a.w_dtype, a.w_vec != 0, a.bias != nullptr, w, bvv);
    const float bv = bvv[0];

    // history of the segment's first vector (only lane 0's copy is consumed)
    float carry[3] = {0.0f, 0.0f, 0.0f};
    if (lane == 0) {
        if (seg > 0) {
            const int64_t t0 = (int64_t)v0 * E;
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                float v = load1<DT>(xrow, t0 - 3 + j);
                if constexpr (MASK)
                    v = mul_round<DT>(v, load_mask(a.mask, b * a.m_sb + (t0 - 3 + j) * a.m_sl, a.mask_dtype));
                carry[j] = v;
            }
        } else if (a.init) {
#pragma unroll
            for (int j = 0; j < 3; ++j)
                if (j >= 3 - (W - 1))
                    carry[j] = load1<DT>(a.init, b * a.i_sb + c * a.i_sc + (int64_t)(a.S_in - 3 + j) * a.i_ss);
        }
    }

#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t v = v0 + u * 64u;
        float xr[E], xm_store[MASK ? E : 1];
        float *xm = MASK ? xm_store : xr;
        unpack_vec<DT>(X[u], xr);
        if constexpr (MASK) {
#pragma unroll
            for (int j = 0; j < E; ++j) xm[j] = mul_round<DT>(xr[j], M[u][j]);
        }
        // seq[0..2] = the three masked inputs before this vector
        float seq[E + 3];
        seq[0] = wave_shift_up(xm[E - 3], carry[0]);
        seq[1] = wave_shift_up(xm[E - 2], carry[1]);
        seq[2] = wave_shift_up(xm[E - 1], carry[2]);
        if (u + 1 < U) {
            carry[0] = read_lane63(xm[E - 3]);
            carry[1] = read_lane63(xm[E - 2]);
            carry[2] = read_lane63(xm[E - 1]);
        }
#pragma unroll
        for (int j = 0; j < E; ++j) seq[3 + j] = xm[j];

        float o[E];
#pragma unroll
        for (int j = 0; j < E; ++j) {
            float acc = bv;
#pragma unroll
            for (int k = 0; k < W; ++k) acc = fmaf(w[0][k], seq[j + (4 - W) + k], acc);
            o[j] = acc;
        }
        if (a.act) {
#pragma unroll
            for (int j = 0; j < E; ++j) o[j] = silu_fast(o[j]);
        }
        if (a.res_mode == CANON_RESIDUAL_UNMASKED || (!MASK && a.res_mode)) {
#pragma unroll
            for (int j = 0; j < E; ++j) o[j] += xr[j];
        } else if (a.res_mode == CANON_RESIDUAL_MASKED) {
#pragma unroll
            for (int j = 0; j < E; ++j) o[j] += xm[j];
        }
        if (v < a.nvec) store_vec<NT>(orow + (int64_t)v * 16, pack_vec<DT>(o));
    }

    if (a.fin && seg == a.nseg - 1) capture_row_state<DT>(a, b, c, lane);
}

// ---------------------------------------------------------------------------
// prefill, channel-contiguous rows ([B, L, C] memory, x_stride_c == 1): the
// layout CanonLayer hands over (a transposed view of [B, T, D]).
//
// One lane owns E adjacent channels (VB = 8 bytes of every row: 4 x 16-bit or
// 2 x fp32; 16-byte lanes need 142 registers and measured 4-9 % slower) and R
// consecutive time steps; the four waves of a block own four consecutive
// R-row slabs of the same 64-lane channel tile, so a block streams a
// [4R rows] x [512 B] tile and consecutive blocks sweep memory in address
// order (short-lived waves over a compact window: measured to be what HBM
// wants; long per-lane time runs lose 10-20 %).  The three rows a wave needs from before its slab are the
// last three rows of the previous wave: each wave publishes the raw tail of
// its slab in LDS, one barrier, the next wave picks it up -- only the first
// wave of a block reads its halo from memory.  All loads (slab, halo, taps)
// are issued before the first wait.
// ---------------------------------------------------------------------------
// keep0..2 (wave uniform): whether the rows t-3, t-2, t-1 belong to the packed sequence of row t
// (always true without seq_idx); a row of another sequence enters as zeros.
template <int DT, int W, bool MASK, bool NT, int VB>
__device__ __forceinline__ void blc_row(const FwdArgs &a, const float (*w)[W], const float *bias,
                                        float (*hist)[VB / Elem<DT>::bytes], const typename VecIO<VB>::type &X, float m,
                                        char *optr, bool active, bool keep0 = true, bool keep1 = true, bool keep2 = true)
{
    constexpr int E = VB / Elem<DT>::bytes;
    float xr[E], xm_store[MASK ? E : 1], o[E];
    float *xm = MASK ? xm_store : xr;
    VecIO<VB>::template unpack<DT>(X, xr);
    if constexpr (MASK) {
#pragma unroll
        for (int e = 0; e < E; ++e) xm[e] = mul_round<DT>(xr[e], m);
    }
#pragma unroll
    for (int e = 0; e < E; ++e) {
        float acc = bias[e];
        if constexpr (W == 4) acc = fmaf(w[e][0], keep0 ? hist[0][e] : 0.0f, acc);
        if constexpr (W >= 3) acc = fmaf(w[e][W - 3], keep1 ? hist[1][e] : 0.0f, acc);
        acc = fmaf(w[e][W - 2], keep2 ? hist[2][e] : 0.0f, acc);
        acc = fmaf(w[e][W - 1], xm[e], acc);
        o[e] = acc;
        hist[0][e] = hist[1][e];
        hist[1][e] = hist[2][e];
        hist[2][e] = xm[e];
    }
    if (a.act) {
#pragma unroll
        for (int e = 0; e < E; ++e) o[e] = silu_fast(o[e]);
    }
    if (a.res_mode == CANON_RESIDUAL_UNMASKED || (!MASK && a.res_mode)) {
#pragma unroll
        for (int e = 0; e < E; ++e) o[e] += xr[e];
    } else if (a.res_mode == CANON_RESIDUAL_MASKED) {
#pragma unroll
        for (int e = 0; e < E; ++e) o[e] += xm[e];
    }
    if (active) VecIO<VB>::template store<NT>(optr, VecIO<VB>::template pack<DT>(o));
}

constexpr int kBlcWaves = 4;   // waves (time slabs) per block
constexpr int kBlcVecBytes = 8;   // bytes per lane and access: 8 measured 4-9 % faster than 16 (half the registers, twice the waves)

template <int DT, int W, int R, bool MASK, bool NT, bool SEQ = false, int VB = kBlcVecBytes>
__device__ __forceinline__ void blc_block(const FwdArgs &a, const uint32_t blk)
{
    constexpr int E = VB / Elem<DT>::bytes;
    using V = VecIO<VB>;
    using vec_t = typename V::type;
    static_assert(R >= 3, "a slab must hold the three rows the next slab needs");
    __shared__ vec_t tail[kBlcWaves][3][64];   // raw last three rows of each wave's slab

    // blocks in plain memory order (an XCD-contiguous remap measured 3 % slower here)
    // blk = (b * ntt + tt) * nct + ct : channel tile fastest, i.e. memory order
    const uint32_t bt = fdiv(blk, a.div_nct);
    const uint32_t ct = blk - bt * a.nct;
    const uint32_t b = fdiv(bt, a.div_ntt);
    const uint32_t tt = bt - b * a.ntt;
    const int lane = threadIdx.x & 63;
    const uint32_t wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t cv = ct * 64u + lane;
    const bool active = cv < a.nvec;
    const uint32_t c0 = (active ? cv : a.nvec - 1u) * E;   // idle lanes shadow the last vector, loads need no predicate

    const char *xb = a.x + ((int64_t)b * a.x_sb + c0) * Elem<DT>::bytes;
    char *ob = a.out + ((int64_t)b * a.o_sb + c0) * Elem<DT>::bytes;
    const int64_t xs = a.x_sl * Elem<DT>::bytes, os = a.o_sl * Elem<DT>::bytes;
    const int64_t t0 = ((int64_t)tt * kBlcWaves + wv) * R;
    const int64_t left = (int64_t)a.L - t0;
    const int rows = left >= R ? R : (left > 0 ? (int)left : 0);   // wave uniform
    const int64_t t_last = (int64_t)a.L - 1;

    // slab rows, then (first wave only) the three rows before the block, then the taps.
    // Rows past the end of the sequence are clamped to the last row (loaded, never used).
    vec_t X[R], H[3];
    float m[R], mh[3];
    int32_t sq[SEQ ? R + 3 : 1];   // sequence index of rows t0-3 .. t0+R-1
    RawTaps<E> raw;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        X[r] = V::zero();
        m[r] = 0.0f;
    }
#pragma unroll
    for (int j = 0; j < (SEQ ? R + 3 : 1); ++j) sq[j] = 0;
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        H[j] = V::zero();
        mh[j] = 0.0f;
    }
    if (rows > 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int64_t t = t0 + r < t_last ? t0 + r : t_last;
            X[r] = V::template load<NT>(xb + t * xs);
        }
        if (wv == 0) {
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                const int64_t t = t0 - 3 + j;
                if (j >= 3 - (W - 1) && t >= 0) H[j] = V::template load<false>(xb + t * xs);
            }
        }
        // every wave fetches the taps itself (cache hits); sharing them through LDS was measured slower
        fetch_taps<W, E>(a.weight, a.bias, a.w_sc, a.w_sk, a.w_dtype, a.w_vec != 0, false, c0, raw);
        if constexpr (SEQ) load_seq_rows<R + 3>(a.seq, (int64_t)b * a.q_sb, t0 - 3, a.L, a.q_sl, sq);
        if constexpr (MASK) {
            // mask of the three rows before the slab and of the slab, last so that nothing is issued after its wait
            float mm[R + 3];
            load_mask_rows<R + 3>(a.mask, (int64_t)b * a.m_sb, t0 - 3, a.L, a.m_sl, a.mask_dtype, mm);
#pragma unroll
            for (int j = 0; j < 3; ++j) mh[j] = mm[j];
#pragma unroll
            for (int r = 0; r < R; ++r) m[r] = mm[3 + r];
        }
    }

    // hand the raw tail of this slab to the next wave
#pragma unroll
    for (int j = 0; j < 3; ++j) tail[wv][j][lane] = X[R - 3 + j];
    __syncthreads();
    if (wv > 0) {
#pragma unroll
        for (int j = 0; j < 3; ++j)
            if (j >= 3 - (W - 1)) H[j] = tail[wv - 1][j][lane];
    }
    if (rows == 0) return;   // after the barrier

    // hist[j] = masked row t0 - 3 + j
    float hist[3][E];
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        V::template unpack<DT>(H[j], hist[j]);
        if constexpr (MASK) {
#pragma unroll
            for (int e = 0; e < E; ++e) hist[j][e] = mul_round<DT>(hist[j][e], mh[j]);
        }
    }
    if (t0 == 0 && a.init && active) {
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            if (j < 3 - (W - 1)) continue;
#pragma unroll
            for (int e = 0; e < E; ++e)
                hist[j][e] = load1<DT>(a.init, b * a.i_sb + (int64_t)(c0 + e) * a.i_sc + (int64_t)(a.S_in - 3 + j) * a.i_ss);
        }
    }
    float w[E][W], bias[E];
    decode_taps<DT, W, E>(raw, a.w_dtype, a.w_vec != 0, a.bias != nullptr, w, bias);

    if constexpr (SEQ) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (r >= rows) continue;
            // rows t-3, t-2, t-1 count only if they carry the index of row t; sequence boundaries are rare,
            // so the all-kept case takes the plain code
            const int32_t cur = sq[3 + r];
            const bool k0 = sq[r] == cur, k1 = sq[r + 1] == cur, k2 = sq[r + 2] == cur;
            if (k0 && k1 && k2) blc_row<DT, W, MASK, NT, VB>(a, w, bias, hist, X[r], m[r], ob + (t0 + r) * os, active);
            else blc_row<DT, W, MASK, NT, VB>(a, w, bias, hist, X[r], m[r], ob + (t0 + r) * os, active, k0, k1, k2);
        }
    } else if (rows == R) {
#pragma unroll
        for (int r = 0; r < R; ++r) blc_row<DT, W, MASK, NT, VB>(a, w, bias, hist, X[r], m[r], ob + (t0 + r) * os, active);
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r)
            if (r < rows) blc_row<DT, W, MASK, NT, VB>(a, w, bias, hist, X[r], m[r], ob + (t0 + r) * os, active);
    }

    if (a.fin && active && t0 + rows == (int64_t)a.L) {
        for (int slot = 0; slot < a.S_out; ++slot) {
            const int64_t t = (int64_t)a.L - a.S_out + slot;
            float v[E];
#pragma unroll
            for (int e = 0; e < E; ++e) v[e] = 0.0f;
            if (t >= 0) {
                V::template unpack<DT>(V::template load<false>(xb + t * xs), v);
                if constexpr (MASK) {
                    const float mm = load_mask(a.mask, b * a.m_sb + t * a.m_sl, a.mask_dtype);
#pragma unroll
                    for (int e = 0; e < E; ++e) v[e] = mul_round<DT>(v[e], mm);
                }
            } else if (a.init && a.S_in + t >= 0) {
#pragma unroll
                for (int e = 0; e < E; ++e)
                    v[e] = load1<DT>(a.init, b * a.i_sb + (int64_t)(c0 + e) * a.i_sc + (a.S_in + t) * a.i_ss);
            }
#pragma unroll
            for (int e = 0; e < E; ++e)
                store1<DT>(a.fin, b * a.f_sb + (int64_t)(c0 + e) * a.f_sc + slot * a.f_ss, v[e]);
        }
    }
}

template <int DT, int W, int R, bool MASK, bool NT>
__global__ __launch_bounds__(256) void canon_fwd_blc_kernel(const FwdArgs a)
{
    blc_block<DT, W, R, MASK, NT>(a, blockIdx.x);
}

// the same over packed variable-length sequences (seq_idx)
template <int DT, int W, int R, bool MASK>
__global__ __launch_bounds__(256) void canon_fwd_blc_seq_kernel(const FwdArgs a)
{
    blc_block<DT, W, R, MASK, false, true, kBlcVecBytes>(a, blockIdx.x);
}

// Several channel ranges of one logical [B, C, L] problem that live in separate
// tensors (q / k / v or gate / up projections), one launch: every block belongs
// to one part and runs the single-tensor code on that part's argument block.
constexpr int kMaxParts = CANON_CONV1D_MAX_PARTS;

template <typename Args> struct PartTable {
    Args part[kMaxParts];
    uint32_t first_block[kMaxParts];   // first block of each part; 0xFFFFFFFF for unused slots
};

template <typename Args>
__device__ __forceinline__ uint32_t part_of_block(const PartTable<Args> &m, uint32_t blk)
{
    uint32_t p = 0;
#pragma unroll
    for (int i = 1; i < kMaxParts; ++i) p += blk >= m.first_block[i] ? 1u : 0u;
    return p;
}

template <int DT, int W, int R, bool MASK, bool NT>
__global__ __launch_bounds__(256) void canon_fwd_blc_parts_kernel(const PartTable<FwdArgs> m)
{
    const uint32_t p = part_of_block(m, blockIdx.x);
    blc_block<DT, W, R, MASK, NT>(m.part[p], blockIdx.x - m.first_block[p]);
}

// ---------------------------------------------------------------------------
// prefill, any strides / any length / either rounding mode: one thread per
// (b, c, chunk of time steps), scalar accesses.
// ---------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(256) void canon_fwd_generic_kernel(const FwdArgs a)
{
    const uint64_t tid = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (tid >= a.ntasks) return;
    // fastest-varying index follows the contiguous dimension of x
    uint32_t b, c, ch;
    if (a.x_sc == 1 && a.x_sl != 1) {
        c = tid % a.C;
        const uint32_t r = tid / a.C;
        ch = r % a.nseg;
        b = r / a.nseg;
    } else {
        ch = tid % a.nseg;
        const uint32_t r = tid / a.nseg;
        c = r % a.C;
        b = r / a.C;
    }
    const int W = a.W;
    float w[4] = {0, 0, 0, 0};
    for (int k = 0; k < W; ++k)
        w[4 - W + k] = round_through<DT>(load_w(a.weight, (int64_t)c * a.w_sc + k * a.w_sk, a.w_dtype));
    const float bv = a.bias ? round_through<DT>(load_w(a.bias, c, a.w_dtype)) : 0.0f;

    const int64_t xo = (int64_t)b * a.x_sb + (int64_t)c * a.x_sc;
    const int64_t oo = (int64_t)b * a.o_sb + (int64_t)c * a.o_sc;
    const int64_t t_begin = (int64_t)ch * a.chunk;
    const int64_t t_stop = t_begin + (int64_t)a.chunk;
    const int64_t t_end = t_stop < (int64_t)a.L ? t_stop : (int64_t)a.L;

    float h[3] = {0, 0, 0};
    int32_t qh[3] = {0, 0, 0};   // with seq_idx: the sequence each history position belongs to
    const int32_t *seq = a.seq ? a.seq + (int64_t)b * a.q_sb : nullptr;
    for (int j = 4 - W; j < 3; ++j) {
        const int64_t t = t_begin - 3 + j;
        if (t >= 0) {
            float v = load1<DT>(a.x, xo + t * a.x_sl);
            if (a.mask) v = mul_round<DT>(v, load_mask(a.mask, b * a.m_sb + t * a.m_sl, a.mask_dtype));
            h[j] = v;
            if (seq) qh[j] = seq[t * a.q_sl];
        } else if (a.init && a.S_in + t >= 0) {
            h[j] = load1<DT>(a.init, b * a.i_sb + c * a.i_sc + (a.S_in + t) * a.i_ss);
        }
    }
    for (int64_t t = t_begin; t < t_end; ++t) {
        const float xr = load1<DT>(a.x, xo + t * a.x_sl);
        float xm = xr;
        if (a.mask) xm = mul_round<DT>(xr, load_mask(a.mask, b * a.m_sb + t * a.m_sl, a.mask_dtype));
        float acc = bv;
        if (seq) {
            // inputs of another packed sequence enter as zeros
            const int32_t qt = seq[t * a.q_sl];
            if (W == 4) acc = fmaf(w[0], qh[0] == qt ? h[0] : 0.0f, acc);
            if (W >= 3) acc = fmaf(w[1], qh[1] == qt ? h[1] : 0.0f, acc);
            acc = fmaf(w[2], qh[2] == qt ? h[2] : 0.0f, acc);
            acc = fmaf(w[3], xm, acc);
            qh[0] = qh[1];
            qh[1] = qh[2];
            qh[2] = qt;
        } else {
            if (W == 4) acc = fmaf(w[0], h[0], acc);
            if (W >= 3) acc = fmaf(w[1], h[1], acc);
            acc = fmaf(w[2], h[2], acc);
            acc = fmaf(w[3], xm, acc);
        }
        if (a.eager) {
            acc = round_through<DT>(acc);
            if (a.act) acc = round_through<DT>(silu_precise(acc));
            if (a.res_mode == CANON_RESIDUAL_MASKED) acc += xm;
            else if (a.res_mode == CANON_RESIDUAL_UNMASKED) acc += xr;
        } else {
            acc = finish(acc, a.act, a.res_mode, xm, xr);
        }
        store1<DT>(a.out, oo + t * a.o_sl, acc);
        h[0] = h[1];
        h[1] = h[2];
        h[2] = xm;
    }
    if (a.fin && ch == a.nseg - 1)
        for (int slot = 0; slot < a.S_out; ++slot) capture_row_state<DT>(a, b, c, slot);
}

// ---------------------------------------------------------------------------
// backward of the prefill: dx, and per-chunk partial sums of dweight / dbias
//
// One lane owns E channels and walks a chunk of time steps from its END to its
// start: dx[t] needs dz[t .. t+W-1] (the three later steps are carried in
// registers), z[t] needs xm[t-3 .. t] (a sliding window refilled with one row
// per step, fetched R rows ahead).  The three dz values just past the chunk are
// recomputed from memory.  dweight / dbias accumulate in registers over the
// chunk and go to partial[(b * nchunk + chunk) * C + c][5] (w0..w3, bias);
// canon_bwd_reduce_kernel sums the partial sets in a fixed order.
//   VEC:  channel-contiguous tensors, E = elements per 16 bytes, vector access
//   !VEC: E = 1, any strides (the fallback for every other layout)
// ---------------------------------------------------------------------------
struct BwdArgs {
    const char *x;
    const char *dy;
    char *dx;
    const void *weight;
    const void *bias;
    const void *mask;
    float *partial;
    float *dweight;
    float *dbias;
    int64_t x_sb, x_sc, x_sl;
    int64_t g_sb, g_sc, g_sl;
    int64_t d_sb, d_sc, d_sl;
    int64_t w_sc, w_sk;
    int64_t m_sb, m_sl;
    uint32_t B, C, L;
    int32_t W, w_dtype, mask_dtype, act, res_mode, w_vec, b_vec, b_pair, m_vec;
    uint32_t nvec;      // channel groups per row (C / E)
    uint32_t nchunk;    // time chunks per sequence
    uint32_t chunk;     // time steps per chunk
    uint32_t nthreads;
    uint32_t nsets;     // partial sets = B * nchunk
    uint32_t nct;       // blc: channel tiles per row
    FastDiv div_nvec, div_nchunk, div_nct;
};

__device__ __forceinline__ float silu_grad(float z)
{
    const float s = __builtin_amdgcn_rcpf(1.0f + __expf(-z));
    return s * (1.0f + z * (1.0f - s));
}

template <int DT, int E, bool VEC>
__device__ __forceinline__ void bwd_load_row(const char *base, int64_t row_off, int64_t sc, float *f)
{
    // E values of one time step; VEC: 16 contiguous bytes at base + row_off (bytes)
    if constexpr (VEC) {
        unpack_vec<DT>(load_vec<false>(base + row_off), f);
    } else {
        f[0] = load1<DT>(base + row_off, 0);
    }
}

template <int DT, int W, int E, bool VEC, bool MASK, int R>
__global__ __launch_bounds__(256) void canon_bwd_walk_kernel(const BwdArgs a)
{
    constexpr int BY = Elem<DT>::bytes;
    const uint32_t tid = blockIdx.x * 256u + threadIdx.x;
    if (tid >= a.nthreads) return;
    const uint32_t bc = fdiv(tid, a.div_nvec);
    const uint32_t cv = tid - bc * a.nvec;
    const uint32_t b = fdiv(bc, a.div_nchunk);
    const uint32_t ch = bc - b * a.nchunk;
    const uint32_t c0 = cv * E;

    const char *xb = a.x + ((int64_t)b * a.x_sb + (int64_t)c0 * a.x_sc) * BY;
    const char *gb = a.dy + ((int64_t)b * a.g_sb + (int64_t)c0 * a.g_sc) * BY;
    char *db_ = a.dx + ((int64_t)b * a.d_sb + (int64_t)c0 * a.d_sc) * BY;
    const int64_t xs = a.x_sl * BY, gs = a.g_sl * BY, ds = a.d_sl * BY;
    const int64_t t_begin = (int64_t)ch * a.chunk;
    const int64_t t_stop = t_begin + (int64_t)a.chunk;
    const int64_t t_end = t_stop < (int64_t)a.L ? t_stop : (int64_t)a.L;
    const int64_t Lm1 = (int64_t)a.L - 1;

    RawTaps<E> raw;
    fetch_taps<W, E>(a.weight, a.bias, a.w_sc, a.w_sk, a.w_dtype, VEC && a.w_vec != 0, VEC && a.b_vec != 0, c0, raw);

    // rows t_end-4 .. t_end+2 of xm (window for the last step + the three steps past the chunk)
    float xr7[7][E], m7[7];
#pragma unroll
    for (int j = 0; j < 7; ++j) {
        const int64_t t = t_end - 4 + j;
        const int64_t tc = t < 0 ? 0 : (t > Lm1 ? Lm1 : t);
        bwd_load_row<DT, E, VEC>(xb, tc * xs, a.x_sc, xr7[j]);
        m7[j] = 1.0f;
    }
    float g3[3][E];
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        const int64_t t = t_end + j;
        bwd_load_row<DT, E, VEC>(gb, (t > Lm1 ? Lm1 : t) * gs, a.g_sc, g3[j]);
    }
    if constexpr (MASK) load_mask_rows<7>(a.mask, (int64_t)b * a.m_sb, t_end - 4, a.L, a.m_sl, a.mask_dtype, m7);

    float w[E][W], bias[E];
    decode_taps<DT, W, E>(raw, a.w_dtype, VEC && a.w_vec != 0, a.bias != nullptr, w, bias);

#pragma unroll
    for (int j = 0; j < 7; ++j) {
        const int64_t t = t_end - 4 + j;
        const bool inside = t >= 0 && t <= Lm1;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float v = MASK ? mul_round<DT>(xr7[j][e], m7[j]) : xr7[j][e];
            xr7[j][e] = inside ? v : 0.0f;
        }
    }
    // dzf[j] = dz[t_end + j]
    float dzf[3][E];
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        const bool inside = t_end + j <= Lm1;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float z = bias[e];
#pragma unroll
            for (int k = 0; k < W; ++k) z = fmaf(w[e][k], xr7[j + 1 + (4 - W) + k][e], z);   // xm[t_end+j-(W-1)+k]
            const float d = a.act ? g3[j][e] * silu_grad(z) : g3[j][e];
            dzf[j][e] = inside ? d : 0.0f;
        }
    }
    // xw[k] = xm[t-3+k] for the step being processed, starting with t = t_end - 1
    float xw[4][E];
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int e = 0; e < E; ++e) xw[k][e] = xr7[k][e];

    float dw[E][W], dbs[E];
#pragma unroll
    for (int e = 0; e < E; ++e) {
        dbs[e] = 0.0f;
#pragma unroll
        for (int k = 0; k < W; ++k) dw[e][k] = 0.0f;
    }

    for (int64_t t_hi = t_end - 1; t_hi >= t_begin; t_hi -= R) {
        // this batch: steps t_hi, t_hi-1, .., t_hi-R+1; needs dout of those steps and x rows t-4.
        // Rows are kept as loaded (raw) until their step, to keep the register count down.
        typename std::conditional<VEC, uint4, float>::type G[R], XN[R];
        float mk[R], mn[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int64_t t = t_hi - r;
            const int64_t tg = t < 0 ? 0 : t;
            const int64_t tn = t - 4 < 0 ? 0 : t - 4;
            if constexpr (VEC) {
                G[r] = load_vec<false>(gb + tg * gs);
                XN[r] = load_vec<false>(xb + tn * xs);
            } else {
                G[r] = load1<DT>(gb + tg * gs, 0);
                XN[r] = load1<DT>(xb + tn * xs, 0);
            }
            mk[r] = 1.0f;
            mn[r] = 1.0f;
        }
        if constexpr (MASK) {
            // masks of steps t_hi-R+1 .. t_hi (for dx) and of rows t_hi-R-3 .. t_hi-4 (for the window)
            float mm[R + 4];
            load_mask_rows<R + 4>(a.mask, (int64_t)b * a.m_sb, t_hi - R - 3, a.L, a.m_sl, a.mask_dtype, mm);
#pragma unroll
            for (int r = 0; r < R; ++r) {
                mk[r] = mm[R + 3 - r];      // step t_hi - r
                mn[r] = mm[R - 1 - r];      // row  t_hi - r - 4
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int64_t t = t_hi - r;
            if (t < t_begin) break;
            float g[E], xn[E], dz[E], o[E];
            if constexpr (VEC) {
                unpack_vec<DT>(G[r], g);
                unpack_vec<DT>(XN[r], xn);
            } else {
                g[0] = G[r];
                xn[0] = XN[r];
            }
#pragma unroll
            for (int e = 0; e < E; ++e) {
                float z = bias[e];
#pragma unroll
                for (int k = 0; k < W; ++k) z = fmaf(w[e][k], xw[(4 - W) + k][e], z);
                dz[e] = z;
            }
            if (a.act) {
#pragma unroll
                for (int e = 0; e < E; ++e) dz[e] = g[e] * silu_grad(dz[e]);
            } else {
#pragma unroll
                for (int e = 0; e < E; ++e) dz[e] = g[e];
            }
#pragma unroll
            for (int e = 0; e < E; ++e) {
                // dxm[t] = sum_k w[k] * dz[t + (W-1) - k]
                float acc = w[e][W - 1] * dz[e];
                acc = fmaf(w[e][W - 2], dzf[0][e], acc);
                if constexpr (W >= 3) acc = fmaf(w[e][W - 3], dzf[1][e], acc);
                if constexpr (W == 4) acc = fmaf(w[e][0], dzf[2][e], acc);
                o[e] = acc;
#pragma unroll
                for (int k = 0; k < W; ++k) dw[e][k] = fmaf(dz[e], xw[(4 - W) + k][e], dw[e][k]);
                dbs[e] += dz[e];
                dzf[2][e] = dzf[1][e];
                dzf[1][e] = dzf[0][e];
                dzf[0][e] = dz[e];
            }
            if (a.res_mode == CANON_RESIDUAL_MASKED) {
#pragma unroll
                for (int e = 0; e < E; ++e) o[e] += g[e];
            }
            if constexpr (MASK) {
#pragma unroll
                for (int e = 0; e < E; ++e) o[e] *= mk[r];
            }
            if (a.res_mode == CANON_RESIDUAL_UNMASKED) {
#pragma unroll
                for (int e = 0; e < E; ++e) o[e] += g[e];
            }
            // slide the window one step back: the new oldest row is t - 4
            const bool has_row = t - 4 >= 0;
#pragma unroll
            for (int e = 0; e < E; ++e) {
                float v = xn[e];
                if constexpr (MASK) v = mul_round<DT>(v, mn[r]);
                xw[3][e] = xw[2][e];
                xw[2][e] = xw[1][e];
                xw[1][e] = xw[0][e];
                xw[0][e] = has_row ? v : 0.0f;
            }
            if constexpr (VEC) {
                store_vec<false>(db_ + t * ds, pack_vec<DT>(o));
            } else {
                store1<DT>(db_ + t * ds, 0, o[0]);
            }
        }
    }

    float *pp = a.partial + (((int64_t)b * a.nchunk + ch) * a.C + c0) * 5;
#pragma unroll
    for (int e = 0; e < E; ++e) {
#pragma unroll
        for (int k = 0; k < 4; ++k) pp[e * 5 + k] = k < W ? dw[e][k] : 0.0f;
        pp[e * 5 + 4] = dbs[e];
    }
}

// ---------------------------------------------------------------------------
// backward, channel-contiguous tensors ([B, L, C] viewed as [B, C, L]).
//
// A block is four waves; a lane owns the channels of one 8-byte group (4 x
// 16-bit or 2 x fp32), a wave a slab of kBwdSlab consecutive time steps of a
// 64-lane channel tile, the four waves four consecutive slabs, and the block
// walks over the `chunk` time steps of its chunk one such 32-step tile at a
// time, keeping its dweight / dbias sums in registers.
//
// Per tile, all rows of x and dout of the slab are requested before anything
// is waited for.  The three rows of x before a slab come from the previous
// wave's slab through LDS (the first wave reads them from memory).  dz of the
// slab's first three steps is computed first and handed to the previous wave
// through LDS (that wave's dx needs dz of the three steps after its slab; the
// last wave recomputes them from three extra rows of x and dout).  The slab is
// then swept from its last step to its first:
//   dz[t] = dout[t] * act'(z[t]),  dx[t] = sum_k w[k] * dz[t + (W-1) - k]
// At the end the four waves' sums are added in a fixed order through LDS and
// written as one partial set entry per channel.
// ---------------------------------------------------------------------------
constexpr int kBwdSlab = 8;    // time steps per wave and tile
constexpr int kBwdWaves = 4;

template <int DT> __device__ __forceinline__ void unpack_half(const uint2 &v, float *f)
{
    if constexpr (DT == CANON_DTYPE_F32) {
        f[0] = bits_f(v.x);
        f[1] = bits_f(v.y);
    } else {
        unpack2<DT>(v.x, f[0], f[1]);
        unpack2<DT>(v.y, f[2], f[3]);
    }
}

template <int DT> __device__ __forceinline__ uint2 pack_half(const float *f)
{
    if constexpr (DT == CANON_DTYPE_F32) return make_uint2(f_bits(f[0]), f_bits(f[1]));
    else return make_uint2(pack2<DT>(f[0], f[1]), pack2<DT>(f[2], f[3]));
}

// One raw row -> the bits of xm = x * mask in the storage type (zero when the row does not exist)
template <int DT, bool MASK>
__device__ __forceinline__ uint2 bwd_mask_row(const uint2 &raw, float m, bool exists)
{
    uint2 v = raw;
    if constexpr (MASK) {
        if constexpr (DT == CANON_DTYPE_F32) {
            v.x = f_bits(bits_f(raw.x) * m);
            v.y = f_bits(bits_f(raw.y) * m);
        } else {
            float f[4];
            unpack_half<DT>(raw, f);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                f[e] *= m;
                if constexpr (DT == CANON_DTYPE_F16) asm volatile("" : "+v"(f[e]));   // see mul_round
            }
            v = pack_half<DT>(f);
        }
    }
    if (!exists) v = make_uint2(0, 0);
    return v;
}

// dz of one step from its window of xm rows and dout
template <int W, int E, bool ACT>
__device__ __forceinline__ void bwd_dz(const float (*w)[W], const float *bias, const float *x0, const float *x1,
                                       const float *x2, const float *x3, const float *g, float *dz)
{
    if constexpr (ACT) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float z = bias[e];
            if constexpr (W == 4) z = fmaf(w[e][0], x0[e], z);
            if constexpr (W >= 3) z = fmaf(w[e][W - 3], x1[e], z);
            z = fmaf(w[e][W - 2], x2[e], z);
            z = fmaf(w[e][W - 1], x3[e], z);
            dz[e] = g[e] * silu_grad(z);
        }
    } else {
#pragma unroll
        for (int e = 0; e < E; ++e) dz[e] = g[e];
    }
}

// The sweep over one slab, last step first.  X / H hold xm in storage bits, dzh the dz of the
// first three steps (already zero past the end of the sequence), dzf the dz of the three steps
// after the slab.  FULL: all R steps exist.
template <int DT, int W, bool MASK, bool ACT, bool FULL, int R, int E>
__device__ __forceinline__ void bwd_sweep(const BwdArgs &a, const float (*w)[W], const float *bias, const uint2 *X,
                                          const uint2 *H, const uint2 *G, const float *mm, const float (*dzh)[E],
                                          float (*dzf)[E], float (*dw)[W], float *dbs, char *dxp, int64_t ds, int rows,
                                          bool active)
{
    float xw[4][E];   // xm of rows r-3 .. r
#pragma unroll
    for (int k = 0; k < 4; ++k) unpack_half<DT>(X[R - 4 + k], xw[k]);
#pragma unroll
    for (int r = R - 1; r >= 0; --r) {
        float g[E], dz[E], o[E];
        unpack_half<DT>(G[r], g);
        if (r >= 3) {
            bwd_dz<W, E, ACT>(w, bias, xw[0], xw[1], xw[2], xw[3], g, dz);
            if constexpr (!FULL) {
#pragma unroll
                for (int e = 0; e < E; ++e) dz[e] = r < rows ? dz[e] : 0.0f;
            }
        } else {
#pragma unroll
            for (int e = 0; e < E; ++e) dz[e] = dzh[r][e];
        }
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float acc = w[e][W - 1] * dz[e];
            acc = fmaf(w[e][W - 2], dzf[0][e], acc);
            if constexpr (W >= 3) acc = fmaf(w[e][W - 3], dzf[1][e], acc);
            if constexpr (W == 4) acc = fmaf(w[e][0], dzf[2][e], acc);
            o[e] = acc;
#pragma unroll
            for (int k = 0; k < W; ++k) dw[e][k] = fmaf(dz[e], xw[(4 - W) + k][e], dw[e][k]);
            dbs[e] += dz[e];
            dzf[2][e] = dzf[1][e];
            dzf[1][e] = dzf[0][e];
            dzf[0][e] = dz[e];
        }
        if (a.res_mode == CANON_RESIDUAL_MASKED) {
#pragma unroll
            for (int e = 0; e < E; ++e) o[e] += g[e];
        }
        if constexpr (MASK) {
#pragma unroll
            for (int e = 0; e < E; ++e) o[e] *= mm[3 + r];
        }
        if (a.res_mode == CANON_RESIDUAL_UNMASKED) {
#pragma unroll
            for (int e = 0; e < E; ++e) o[e] += g[e];
        }
        if ((FULL || r < rows) && active) *(uint2 *)(dxp + r * ds) = pack_half<DT>(o);
        if (r > 0) {
            // slide the window one step back: the new oldest row is r - 4
#pragma unroll
            for (int e = 0; e < E; ++e) {
                xw[3][e] = xw[2][e];
                xw[2][e] = xw[1][e];
                xw[1][e] = xw[0][e];
            }
            unpack_half<DT>(r - 4 >= 0 ? X[r - 4 >= 0 ? r - 4 : 0] : H[r - 1 < 3 ? r - 1 : 0], xw[0]);
        }
    }
}

template <int DT, int W, bool MASK, bool ACT>
__global__ __launch_bounds__(256) void canon_bwd_blc_kernel(const BwdArgs a)
{
    constexpr int BY = Elem<DT>::bytes;
    constexpr int E = 8 / BY;
    constexpr int R = kBwdSlab, NW = kBwdWaves;
    __shared__ uint2 tailx[NW][3][64];            // last three xm rows of each wave's slab (storage bits)
    __shared__ float headdz[NW][3][E][64];        // dz of the first three steps of each wave's slab
    __shared__ float red[NW - 1][5 * E][64];      // dweight / dbias sums of waves 1..3

    // blockIdx = (b * nchunk + ch) * nct + ct : channel tile fastest, i.e. memory order
    const uint32_t bc = fdiv(blockIdx.x, a.div_nct);
    const uint32_t ct = blockIdx.x - bc * a.nct;
    const uint32_t b = fdiv(bc, a.div_nchunk);
    const uint32_t ch = bc - b * a.nchunk;
    const int lane = threadIdx.x & 63;
    const uint32_t wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t cv = ct * 64u + lane;
    const bool active = cv < a.nvec;
    const uint32_t c0 = (active ? cv : a.nvec - 1u) * E;   // idle lanes shadow the last group: loads need no predicate

    const char *xb = a.x + ((int64_t)b * a.x_sb + c0) * BY;
    const char *gb = a.dy + ((int64_t)b * a.g_sb + c0) * BY;
    char *db_ = a.dx + ((int64_t)b * a.d_sb + c0) * BY;
    const int64_t xs = a.x_sl * BY, gs = a.g_sl * BY, ds = a.d_sl * BY;
    const int64_t Lm1 = (int64_t)a.L - 1;
    const int64_t t_chunk = (int64_t)ch * a.chunk;
    const int ntiles = (int)(a.chunk / (uint32_t)(R * NW));

    RawTaps<E> rawt;
    fetch_taps<W, E>(a.weight, a.bias, a.w_sc, a.w_sk, a.w_dtype, a.w_vec != 0, false, c0, rawt);
    float w[E][W], bias[E];

    // The tiles are walked from the last to the first, so the dz of the three steps after a tile
    // are the head of the tile done just before (still in headdz[0]).  For the chunk's last tile
    // the last wave computes them here, from six rows of x and three of dout, and leaves them
    // in that slot itself.
    {
        const int64_t te = t_chunk + (int64_t)a.chunk;   // first step after the chunk (at least 32)
        uint2 XE[6], GE[3];
        float me[6];
#pragma unroll
        for (int j = 0; j < 6; ++j) {
            XE[j] = make_uint2(0, 0);
            me[j] = 1.0f;
        }
#pragma unroll
        for (int j = 0; j < 3; ++j) GE[j] = make_uint2(0, 0);
        if (wv == NW - 1 && te <= Lm1) {
#pragma unroll
            for (int j = 0; j < 6; ++j) {
                const int64_t t = te - 3 + j;
                XE[j] = *(const uint2 *)(xb + (t < Lm1 ? t : Lm1) * xs);
            }
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                const int64_t t = te + j;
                GE[j] = *(const uint2 *)(gb + (t < Lm1 ? t : Lm1) * gs);
            }
            if constexpr (MASK) load_mask_rows<6>(a.mask, (int64_t)b * a.m_sb, te - 3, a.L, a.m_sl, a.mask_dtype, me);
        }
        decode_taps<DT, W, E>(rawt, a.w_dtype, a.w_vec != 0, a.bias != nullptr, w, bias);
        if (wv == NW - 1) {
            float xt[6][E];
#pragma unroll
            for (int j = 0; j < 6; ++j) unpack_half<DT>(bwd_mask_row<DT, MASK>(XE[j], me[j], te - 3 + j <= Lm1), xt[j]);
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                float g[E], d[E];
                unpack_half<DT>(GE[j], g);
                bwd_dz<W, E, ACT>(w, bias, xt[j], xt[j + 1], xt[j + 2], xt[j + 3], g, d);
                const bool inside = te + j <= Lm1;
#pragma unroll
                for (int e = 0; e < E; ++e) headdz[0][j][e][lane] = inside ? d[e] : 0.0f;
            }
        }
    }

    float dw[E][W], dbs[E];
#pragma unroll
    for (int e = 0; e < E; ++e) {
        dbs[e] = 0.0f;
#pragma unroll
        for (int k = 0; k < W; ++k) dw[e][k] = 0.0f;
    }

    // rows of x and dout, the three rows of x before the slab (first wave) and the mask entries of one tile;
    // requested one tile ahead, so that they arrive while the tile before is being computed
    uint2 Xn[R], Gn[R], Hn[3];
    float mmn[R + 3];   // mask of steps t0-3 .. t0+R-1
    auto request = [&](int it) {
        const int64_t t0 = t_chunk + ((int64_t)it * NW + wv) * R;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int64_t t = t0 + r < Lm1 ? t0 + r : Lm1;
            Xn[r] = *(const uint2 *)(xb + t * xs);
            Gn[r] = *(const uint2 *)(gb + t * gs);
        }
#pragma unroll
        for (int j = 0; j < 3; ++j) Hn[j] = make_uint2(0, 0);
        if (wv == 0) {
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                const int64_t t = t0 - 3 + j;
                if (t >= 0) Hn[j] = *(const uint2 *)(xb + (t < Lm1 ? t : Lm1) * xs);
            }
        }
#pragma unroll
        for (int j = 0; j < R + 3; ++j) mmn[j] = 1.0f;
        if constexpr (MASK) load_mask_rows<R + 3>(a.mask, (int64_t)b * a.m_sb, t0 - 3, a.L, a.m_sl, a.mask_dtype, mmn);
    };
    request(ntiles - 1);

    for (int it = ntiles - 1; it >= 0; --it) {
        const int64_t t0 = t_chunk + ((int64_t)it * NW + wv) * R;
        const int64_t left = (int64_t)a.L - t0;
        const int rows = left >= R ? R : (left > 0 ? (int)left : 0);   // wave uniform

        uint2 X[R], G[R], H[3];
        float mm[R + 3];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            X[r] = Xn[r];
            G[r] = Gn[r];
        }
#pragma unroll
        for (int j = 0; j < 3; ++j) H[j] = Hn[j];
#pragma unroll
        for (int j = 0; j < R + 3; ++j) mm[j] = mmn[j];
        if (it > 0) request(it - 1);

        // dz of the three steps after the slab; the last wave's are the previous iteration's head of wave 0
        float dzf[3][E];   // dzf[j] = dz[t + 1 + j] for the step t being processed
        if (wv == NW - 1) {
#pragma unroll
            for (int j = 0; j < 3; ++j)
#pragma unroll
                for (int e = 0; e < E; ++e) dzf[j][e] = headdz[0][j][e][lane];
        }

        // ---- rows become xm (masked, zero where they do not exist), once ----------------
        if (MASK || rows < R) {
#pragma unroll
            for (int r = 0; r < R; ++r) X[r] = bwd_mask_row<DT, MASK>(X[r], mm[3 + r], r < rows);
        }
        if constexpr (MASK) {
            if (wv == 0) {
#pragma unroll
                for (int j = 0; j < 3; ++j) H[j] = bwd_mask_row<DT, MASK>(H[j], mm[j], true);   // zero already when t < 0
            }
        }
#pragma unroll
        for (int j = 0; j < 3; ++j) tailx[wv][j][lane] = X[R - 3 + j];
        __syncthreads();
        if (wv > 0) {
#pragma unroll
            for (int j = 0; j < 3; ++j) H[j] = tailx[wv - 1][j][lane];
        }

        // ---- dz of the slab's first three steps, handed to the previous wave ---------
        float dzh[3][E];
        {
            float xq[6][E];   // xm of rows -3 .. 2
#pragma unroll
            for (int k = 0; k < 3; ++k) unpack_half<DT>(H[k], xq[k]);
#pragma unroll
            for (int k = 0; k < 3; ++k) unpack_half<DT>(X[k], xq[3 + k]);
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                float g[E];
                unpack_half<DT>(G[j], g);
                bwd_dz<W, E, ACT>(w, bias, xq[j], xq[j + 1], xq[j + 2], xq[j + 3], g, dzh[j]);
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    dzh[j][e] = j < rows ? dzh[j][e] : 0.0f;
                    headdz[wv][j][e][lane] = dzh[j][e];
                }
            }
        }
        __syncthreads();
        if (wv < NW - 1) {
#pragma unroll
            for (int j = 0; j < 3; ++j)
#pragma unroll
                for (int e = 0; e < E; ++e) dzf[j][e] = headdz[wv + 1][j][e][lane];
        }

        // ---- sweep the slab from its last step to its first --------------------------
        if (rows == R)
            bwd_sweep<DT, W, MASK, ACT, true, R, E>(a, w, bias, X, H, G, mm, dzh, dzf, dw, dbs, db_ + t0 * ds, ds, rows, active);
        else
            bwd_sweep<DT, W, MASK, ACT, false, R, E>(a, w, bias, X, H, G, mm, dzh, dzf, dw, dbs, db_ + t0 * ds, ds, rows, active);
    }

    // ---- the four waves' sums, added in the order 0, 1, 2, 3 -----------------------------
    if (wv > 0) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
#pragma unroll
            for (int k = 0; k < W; ++k) red[wv - 1][e * 5 + k][lane] = dw[e][k];
            red[wv - 1][e * 5 + 4][lane] = dbs[e];
        }
    }
    __syncthreads();
    if (wv == 0 && active) {
        float *pp = a.partial + (((int64_t)b * a.nchunk + ch) * a.C + c0) * 5;
#pragma unroll
        for (int e = 0; e < E; ++e) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                float v = 0.0f;
                if (k < W) {
                    v = dw[e][k < W ? k : 0];
#pragma unroll
                    for (int q = 0; q < NW - 1; ++q) v += red[q][e * 5 + k][lane];
                }
                pp[e * 5 + k] = v;
            }
            float v = dbs[e];
#pragma unroll
            for (int q = 0; q < NW - 1; ++q) v += red[q][e * 5 + 4][lane];
            pp[e * 5 + 4] = v;
        }
    }
}

// ---------------------------------------------------------------------------
// backward, time-contiguous rows ([B, C, L]): one wave owns one segment of one
// (b, c) row, U vectors of E time steps per lane, exactly as the forward
// kernel.  Pass 1 recomputes z and dz = dout * act'(z) for the lane's own
// steps (history from lane l-1 by wave shift) and accumulates the lane's share
// of dweight / dbias; pass 2 forms dx[t] = sum_k w[k] * dz[t+(W-1)-k] with the
// three later dz values taken from lane l+1 (wave shift the other way), from
// the next vector's lane 0, or -- for the last lane of a segment that is not
// the end of the row -- recomputed from memory.  The wave's dweight / dbias
// are reduced across lanes in a fixed butterfly order and written as one
// partial set entry; canon_bwd_reduce_kernel sums the sets.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float wave_shift_down(float v, float last)
{
    // lane i <- lane i+1 across the whole wave; lane 63 <- `last`
    return bits_f((uint32_t)__builtin_amdgcn_update_dpp((int)f_bits(last), (int)f_bits(v),
                                                        0x130 /* wave_shl:1 */, 0xF, 0xF, false));
}

__device__ __forceinline__ float read_lane0(float v)
{
    return bits_f((uint32_t)__builtin_amdgcn_readfirstlane((int)f_bits(v)));
}

__device__ __forceinline__ float wave_sum(float v)
{
    // fixed-order butterfly: every lane ends with the same total
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

template <int DT, int W, int U, bool MASK>
__global__ __launch_bounds__(256) void canon_bwd_bcl_kernel(const BwdArgs a)
{
    constexpr int E = Elem<DT>::per_vec;
    constexpr int BY = Elem<DT>::bytes;
    const int lane = threadIdx.x & 63;
    const uint32_t task = __builtin_amdgcn_readfirstlane(blockIdx.x * 4u + (threadIdx.x >> 6));
    if (task >= a.nthreads) return;          // nthreads = wave tasks in this kernel
    uint32_t row = task, seg = 0;
    if (a.nchunk > 1) {                      // nchunk = segments per row
        row = fdiv(task, a.div_nchunk);
        seg = task - row * a.nchunk;
    }
    const uint32_t b = fdiv(row, a.div_nvec);   // div_nvec divides by C here
    const uint32_t c = row - b * a.C;

    const char *xrow = a.x + ((int64_t)b * a.x_sb + (int64_t)c * a.x_sc) * BY;
    const char *grow = a.dy + ((int64_t)b * a.g_sb + (int64_t)c * a.g_sc) * BY;
    char *drow = a.dx + ((int64_t)b * a.d_sb + (int64_t)c * a.d_sc) * BY;
    const uint32_t nvec = a.L / E;
    const uint32_t v0 = seg * (64u * U) + lane;

    uint4 X[U], G[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t v = v0 + u * 64u;
        const uint32_t vc = v < nvec ? v : nvec - 1u;
        X[u] = load_vec<false>(xrow + (int64_t)vc * 16);
        G[u] = load_vec<false>(grow + (int64_t)vc * 16);
    }
    RawTaps<1> raw;
    fetch_taps_uniform<W>(a.weight, a.bias, a.w_sc, a.w_sk, a.w_dtype, a.w_vec != 0, a.b_pair != 0, c, raw);
    float M[MASK ? U : 1][E];
    if constexpr (MASK) {
        int64_t mbase[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t v = v0 + u * 64u;
            mbase[u] = b * a.m_sb + (int64_t)(v < nvec ? v : nvec - 1u) * E * a.m_sl;
        }
        load_mask_vec<E, U>(a.mask, mbase, a.m_sl, a.mask_dtype, a.m_vec != 0, M);
    }
    float w[1][W], bvv[1];
    decode_taps<DT, W, 1>(raw, a.w_dtype, a.w_vec != 0, a.bias != nullptr, w, bvv);
    const float bv = bvv[0];

    // left history of the segment's first vector (lane 0 only), right dz of its last vector (lane 63 only)
    float carry[3] = {0.0f, 0.0f, 0.0f};
    float edge[3] = {0.0f, 0.0f, 0.0f};
    const int64_t t_seg0 = (int64_t)seg * (64 * U) * E;
    const int64_t t_seg1 = t_seg0 + (int64_t)(64 * U) * E;      // first step after the segment
    if (lane == 0 && seg > 0) {
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            float v = load1<DT>(xrow, t_seg0 - 3 + j);
            if constexpr (MASK) v = mul_round<DT>(v, load_mask(a.mask, b * a.m_sb + (t_seg0 - 3 + j) * a.m_sl, a.mask_dtype));
            carry[j] = v;
        }
    }
    if (lane == 63 && t_seg1 < (int64_t)a.L) {
        // dz[t_seg1 + j], j = 0..2, from x[t_seg1-3 .. t_seg1+2] and dout[t_seg1 .. t_seg1+2]
        float xs6[6];
#pragma unroll
        for (int i = 0; i < 6; ++i) {
            const int64_t t = t_seg1 - 3 + i;
            float v = 0.0f;
            if (t < (int64_t)a.L) {
                v = load1<DT>(xrow, t);
                if constexpr (MASK) v = mul_round<DT>(v, load_mask(a.mask, b * a.m_sb + t * a.m_sl, a.mask_dtype));
            }
            xs6[i] = v;
        }
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            const int64_t t = t_seg1 + j;
            if (t < (int64_t)a.L) {
                float z = bv;
#pragma unroll
                for (int k = 0; k < W; ++k) z = fmaf(w[0][k], xs6[j + (4 - W) + k], z);
                const float g = load1<DT>(grow, t);
                edge[j] = a.act ? g * silu_grad(z) : g;
            }
        }
    }

    // pass 1: dz of the lane's own steps, and its share of dweight / dbias
    float dz[U][E], gg[U][E];
    float dwl[W], dbl = 0.0f;
#pragma unroll
    for (int k = 0; k < W; ++k) dwl[k] = 0.0f;
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const bool valid = v0 + u * 64u < nvec;
        float xr[E], xm_store[MASK ? E : 1];
        float *xm = MASK ? xm_store : xr;
        unpack_vec<DT>(X[u], xr);
        unpack_vec<DT>(G[u], gg[u]);
        if constexpr (MASK) {
#pragma unroll
            for (int j = 0; j < E; ++j) xm[j] = mul_round<DT>(xr[j], M[u][j]);
        }
        float seq[E + 3];
        seq[0] = wave_shift_up(xm[E - 3], carry[0]);
        seq[1] = wave_shift_up(xm[E - 2], carry[1]);
        seq[2] = wave_shift_up(xm[E - 1], carry[2]);
        if (u + 1 < U) {
            carry[0] = read_lane63(xm[E - 3]);
            carry[1] = read_lane63(xm[E - 2]);
            carry[2] = read_lane63(xm[E - 1]);
        }
#pragma unroll
        for (int j = 0; j < E; ++j) seq[3 + j] = xm[j];
#pragma unroll
        for (int j = 0; j < E; ++j) {
            float z = bv;
#pragma unroll
            for (int k = 0; k < W; ++k) z = fmaf(w[0][k], seq[j + (4 - W) + k], z);
            dz[u][j] = z;
        }
        if (a.act) {
#pragma unroll
            for (int j = 0; j < E; ++j) dz[u][j] = gg[u][j] * silu_grad(dz[u][j]);
        } else {
#pragma unroll
            for (int j = 0; j < E; ++j) dz[u][j] = gg[u][j];
        }
        if (!valid) {
#pragma unroll
            for (int j = 0; j < E; ++j) dz[u][j] = 0.0f;
        }
#pragma unroll
        for (int j = 0; j < E; ++j) {
#pragma unroll
            for (int k = 0; k < W; ++k) dwl[k] = fmaf(dz[u][j], seq[j + (4 - W) + k], dwl[k]);
            dbl += dz[u][j];
        }
    }

    // pass 2: dx
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t v = v0 + u * 64u;
        // the three dz values after this vector: lane l+1 of the same step, for lane 63 lane 0 of the next
        float nx[3];
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            const float last = (u + 1 < U) ? read_lane0(dz[u + 1 < U ? u + 1 : u][j]) : edge[j];
            nx[j] = wave_shift_down(dz[u][j], last);
        }
        float dq[E + 3];
#pragma unroll
        for (int j = 0; j < E; ++j) dq[j] = dz[u][j];
        dq[E] = nx[0]; dq[E + 1] = nx[1]; dq[E + 2] = nx[2];
        float o[E];
#pragma unroll
        for (int j = 0; j < E; ++j) {
            float acc = w[0][W - 1] * dq[j];
#pragma unroll
            for (int k = W - 2; k >= 0; --k) acc = fmaf(w[0][k], dq[j + (W - 1) - k], acc);
            o[j] = acc;
        }
        if (a.res_mode == CANON_RESIDUAL_MASKED) {
#pragma unroll
            for (int j = 0; j < E; ++j) o[j] += gg[u][j];
        }
        if constexpr (MASK) {
#pragma unroll
            for (int j = 0; j < E; ++j) o[j] *= M[u][j];
        }
        if (a.res_mode == CANON_RESIDUAL_UNMASKED) {
#pragma unroll
            for (int j = 0; j < E; ++j) o[j] += gg[u][j];
        }
        if (v < nvec) store_vec<false>(drow + (int64_t)v * 16, pack_vec<DT>(o));
    }

    // the wave's dweight / dbias -> partial[(b * nseg + seg) * C + c][5]
    float tot[5];
#pragma unroll
    for (int k = 0; k < 4; ++k) tot[k] = k < W ? wave_sum(dwl[k < W ? k : 0]) : 0.0f;
    tot[4] = wave_sum(dbl);
    if (lane == 0) {
        float *pp = a.partial + (((int64_t)b * a.nchunk + seg) * a.C + c) * 5;
#pragma unroll
        for (int k = 0; k < 5; ++k) pp[k] = tot[k];
    }
}

// dweight[c, k] / dbias[c] = sum over the partial sets, in a fixed order: a block owns 32 adjacent
// (c, j) columns; its 8 slices each sum every 8th set in set order (fp64), then the slices are added
// in slice order.  Reads are 128 contiguous bytes per set and slice.
__global__ __launch_bounds__(256) void canon_zero_kernel(float *p, uint32_t n)
{
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i < n) p[i] = 0.0f;
}

__global__ __launch_bounds__(256) void canon_bwd_reduce_kernel(const float *partial, float *dweight, float *dbias,
                                                              uint32_t C, uint32_t nsets, int W)
{
    __shared__ double part[8][32];
    const uint32_t col = threadIdx.x & 31u, slice = threadIdx.x >> 5;
    const uint32_t ncols = C * 5u;
    const uint32_t i = blockIdx.x * 32u + col;   // (c, j), j in 0..4
    double acc = 0.0;
    if (i < ncols)
        for (uint32_t s = slice; s < nsets; s += 8u) acc += (double)partial[(int64_t)s * ncols + i];
    part[slice][col] = acc;
    __syncthreads();
    if (slice != 0 || i >= ncols) return;
    double total = part[0][col];
#pragma unroll
    for (int k = 1; k < 8; ++k) total += part[k][col];
    const uint32_t c = i / 5u, j = i - c * 5u;
    if (j < 4) {
        if ((int)j < W) dweight[c * W + j] = (float)total;
    } else if (dbias) {
        dbias[c] = (float)total;
    }
}

// ---------------------------------------------------------------------------
// decode update, vectorised: contiguous [B, C, S] state, channel-contiguous
// x / out.  One lane owns E adjacent channels: it reads the E*S state
// elements as S 16-byte vectors (they are one contiguous 16*S-byte run),
// computes E outputs, and writes the run back shifted by one element per
// channel with the new token in the last slot -- one fused gather / shift /
// write, no second pass.  Each lane walks NB batch rows so the taps are
// fetched once per NB tokens.
// ---------------------------------------------------------------------------
template <int DT> struct StateRun {
    // element i of a run of uint4 vectors, as raw bits of the storage type
    static __device__ __forceinline__ uint32_t get(const uint4 *v, int i)
    {
        if constexpr (DT == CANON_DTYPE_F32) {
            const uint4 &q = v[i >> 2];
            const int d = i & 3;
            return d == 0 ? q.x : d == 1 ? q.y : d == 2 ? q.z : q.w;
        } else {
            const uint4 &q = v[i >> 3];
            const int d = (i >> 1) & 3;
            const uint32_t u = d == 0 ? q.x : d == 1 ? q.y : d == 2 ? q.z : q.w;
            return (i & 1) ? (u >> 16) : (u & 0xFFFFu);
        }
    }
    static __device__ __forceinline__ float as_float(uint32_t raw)
    {
        if constexpr (DT == CANON_DTYPE_F32) return bits_f(raw);
        else if constexpr (DT == CANON_DTYPE_BF16) return bits_f(raw << 16);
        else return (float)__builtin_bit_cast(_Float16, (uint16_t)raw);
    }
    static __device__ __forceinline__ uint32_t raw_of(float f)   // exact for values already representable
    {
        if constexpr (DT == CANON_DTYPE_F32) return f_bits(f);
        else if constexpr (DT == CANON_DTYPE_BF16) return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f);
        else return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
    }
};

template <int DT, int W, int S, int NB>
__device__ __forceinline__ void update_vec_block(const UpdArgs &a, const uint32_t blk)
{
    constexpr int E = Elem<DT>::per_vec;
    constexpr int BY = Elem<DT>::bytes;
    const uint32_t tid = blk * 256u + threadIdx.x;
    if (tid >= a.nthreads) return;
    const uint32_t bg = fdiv(tid, a.div_nvec);
    const uint32_t cv = tid - bg * a.nvec;
    const uint32_t c0 = cv * E;

    uint4 X[NB];
    uint4 ST[NB][S];
    float tm[NB];
#pragma unroll
    for (int n = 0; n < NB; ++n) {
        const uint32_t b = bg * NB + n;
        tm[n] = 1.0f;
        if (b < a.B) {
            X[n] = *(const uint4 *)(a.x + ((int64_t)b * a.x_sb + c0) * BY);
            const uint4 *sp = (const uint4 *)(a.state + ((int64_t)b * a.s_sb + (int64_t)c0 * S) * BY);
#pragma unroll
            for (int k = 0; k < S; ++k) ST[n][k] = sp[k];
        }
    }
    RawTaps<E> raw;
    fetch_taps<W, E>(a.weight, a.bias, a.w_sc, a.w_sk, a.w_dtype, a.w_vec != 0, a.b_vec != 0, c0, raw);
    if (a.tmask) {
        // token masks last and in one go (one element-type switch, one wait)
        int64_t mbase[NB];
        float tmv[NB][1];
#pragma unroll
        for (int n = 0; n < NB; ++n) {
            const uint32_t b = bg * NB + n;
            mbase[n] = (int64_t)(b < a.B ? b : a.B - 1u) * a.m_sb;
        }
        load_mask_vec<1, NB>(a.tmask, mbase, 0, a.mask_dtype, false, tmv);
#pragma unroll
        for (int n = 0; n < NB; ++n) tm[n] = tmv[n][0];
    }
    float w[E][W], bias[E];
    decode_taps<DT, W, E>(raw, a.w_dtype, a.w_vec != 0, a.bias != nullptr, w, bias);

#pragma unroll
    for (int n = 0; n < NB; ++n) {
        const uint32_t b = bg * NB + n;
        if (b >= a.B) continue;
        float xr[E], xt[E], o[E];
        unpack_vec<DT>(X[n], xr);
        if (a.tmask) {
#pragma unroll
            for (int e = 0; e < E; ++e) xt[e] = mul_round<DT>(xr[e], tm[n]);
        } else {
#pragma unroll
            for (int e = 0; e < E; ++e) xt[e] = xr[e];
        }
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float acc = bias[e];
#pragma unroll
            for (int k = 0; k < W - 1; ++k)
                acc = fmaf(w[e][k], StateRun<DT>::as_float(StateRun<DT>::get(ST[n], e * S + (S - (W - 1) + k))), acc);
            o[e] = fmaf(w[e][W - 1], xt[e], acc);
        }
        if (a.act) {
#pragma unroll
            for (int e = 0; e < E; ++e) o[e] = silu_fast(o[e]);
        }
        if (a.res_mode == CANON_RESIDUAL_MASKED) {
#pragma unroll
            for (int e = 0; e < E; ++e) o[e] += xt[e];
        } else if (a.res_mode == CANON_RESIDUAL_UNMASKED) {
#pragma unroll
            for (int e = 0; e < E; ++e) o[e] += xr[e];
        }
        *(uint4 *)(a.out + ((int64_t)b * a.o_sb + c0) * BY) = pack_vec<DT>(o);

        // new run: element (e, k) <- old (e, k+1); (e, S-1) <- token
        uint32_t raw[E * S];
#pragma unroll
        for (int e = 0; e < E; ++e) {
#pragma unroll
            for (int k = 0; k < S - 1; ++k) raw[e * S + k] = StateRun<DT>::get(ST[n], e * S + k + 1);
            raw[e * S + S - 1] = StateRun<DT>::get(&X[n], e);   // the token's own bits
        }
        if (a.tmask) {
#pragma unroll
            for (int e = 0; e < E; ++e) raw[e * S + S - 1] = StateRun<DT>::raw_of(xt[e]);
        }
        uint4 *dp = (uint4 *)(a.state + ((int64_t)b * a.s_sb + (int64_t)c0 * S) * BY);
#pragma unroll
        for (int k = 0; k < S; ++k) {
            uint4 q;
            if constexpr (DT == CANON_DTYPE_F32) {
                q.x = raw[4 * k]; q.y = raw[4 * k + 1]; q.z = raw[4 * k + 2]; q.w = raw[4 * k + 3];
            } else {
                q.x = raw[8 * k] | (raw[8 * k + 1] << 16);
                q.y = raw[8 * k + 2] | (raw[8 * k + 3] << 16);
                q.z = raw[8 * k + 4] | (raw[8 * k + 5] << 16);
                q.w = raw[8 * k + 6] | (raw[8 * k + 7] << 16);
            }
            dp[k] = q;
        }
    }
}

template <int DT, int W, int S, int NB>
__global__ __launch_bounds__(256) void canon_update_vec_kernel(const UpdArgs a)
{
    update_vec_block<DT, W, S, NB>(a, blockIdx.x);
}

// the token of one step given as several channel ranges (separate projections), one launch
template <int DT, int W, int S, int NB>
__global__ __launch_bounds__(256) void canon_update_vec_parts_kernel(const PartTable<UpdArgs> m)
{
    const uint32_t p = part_of_block(m, blockIdx.x);
    update_vec_block<DT, W, S, NB>(m.part[p], blockIdx.x - m.first_block[p]);
}

// decode update, any strides / state length / rounding mode: one thread per (b, c)
template <int DT>
__global__ __launch_bounds__(256) void canon_update_generic_kernel(const UpdArgs a)
{
    const uint64_t tid = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (tid >= a.nthreads) return;
    const uint32_t c = tid % a.C;
    const uint32_t b = tid / a.C;
    const int W = a.W, S = a.S;
    float w[4] = {0, 0, 0, 0}, win[4] = {0, 0, 0, 0};
    for (int k = 0; k < W; ++k)
        w[4 - W + k] = round_through<DT>(load_w(a.weight, (int64_t)c * a.w_sc + k * a.w_sk, a.w_dtype));
    const float bv = a.bias ? round_through<DT>(load_w(a.bias, c, a.w_dtype)) : 0.0f;
    const int64_t so = (int64_t)b * a.s_sb + (int64_t)c * a.s_sc;
    const float xr = load1<DT>(a.x, (int64_t)b * a.x_sb + (int64_t)c * a.x_sc);
    float xt = xr;
    if (a.tmask) xt = mul_round<DT>(xr, load_mask(a.tmask, (int64_t)b * a.m_sb, a.mask_dtype));
    for (int k = 0; k < W - 1; ++k) win[4 - W + k] = load1<DT>(a.state, so + (int64_t)(S - (W - 1) + k) * a.s_ss);
    win[3] = xt;
    float acc;
    if (!a.eager) {
        acc = bv;
        if (W == 4) acc = fmaf(w[0], win[0], acc);
        if (W >= 3) acc = fmaf(w[1], win[1], acc);
        acc = fmaf(w[2], win[2], acc);
        acc = fmaf(w[3], win[3], acc);
        acc = finish(acc, a.act, a.res_mode, xt, xr);
    } else {
        float s = 0.0f;
        for (int k = 4 - W; k < 4; ++k) s = __fadd_rn(s, mul_round<DT>(win[k], w[k]));
        s = round_through<DT>(s);
        acc = round_through<DT>(__fadd_rn(bv, s));
        if (a.act) acc = round_through<DT>(silu_precise(acc));
        if (a.res_mode == CANON_RESIDUAL_MASKED) acc = __fadd_rn(acc, xt);
        else if (a.res_mode == CANON_RESIDUAL_UNMASKED) acc = __fadd_rn(acc, xr);
    }
    store1<DT>(a.out, (int64_t)b * a.o_sb + (int64_t)c * a.o_sc, acc);
    // shift left by one (ascending order: each slot is read before it is overwritten)
    for (int k = 0; k < S - 1; ++k) {
        if constexpr (DT == CANON_DTYPE_F32)
            ((uint32_t *)a.state)[so + k * a.s_ss] = ((const uint32_t *)a.state)[so + (k + 1) * a.s_ss];
        else
            ((uint16_t *)a.state)[so + k * a.s_ss] = ((const uint16_t *)a.state)[so + (k + 1) * a.s_ss];
    }
    store1<DT>(a.state, so + (int64_t)(S - 1) * a.s_ss, xt);
}

// ---------------------------------------------------------------------------
// host side: validation, planning, launch
// ---------------------------------------------------------------------------
thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

bool valid_dtype(int d) { return d == CANON_DTYPE_F32 || d == CANON_DTYPE_BF16 || d == CANON_DTYPE_F16; }
bool valid_mask_dtype(int d) { return d >= CANON_MASK_U8 && d <= CANON_MASK_F16; }
int elem_bytes(int d) { return d == CANON_DTYPE_F32 ? 4 : 2; }
bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

FastDiv make_fastdiv(uint32_t d)
{
    // floor(n / d) for 0 <= n < 2^32 (Granlund-Montgomery round-up method)
    FastDiv f;
    f.d = d ? d : 1;
    uint32_t l = 0;
    while ((1ull << l) < f.d) ++l;
    f.m = (uint32_t)(((1ull << 32) * ((1ull << l) - f.d)) / f.d + 1);
    f.s1 = l < 1 ? l : 1;
    f.s2 = l > 0 ? l - 1 : 0;
    return f;
}

// a run of E consecutive mask entries (E = elements of x per 16 bytes) starting
// at a multiple of E is contiguous and aligned to its own size
bool mask_run_aligned(const void *mask, int mask_dtype, int64_t stride_b, int64_t stride_l, int x_dtype)
{
    if (!mask || stride_l != 1) return false;
    static const int msize[] = {1, 4, 8, 4, 2, 2};
    const int E = 16 / elem_bytes(x_dtype);
    const int64_t run = (int64_t)E * msize[mask_dtype];
    const int64_t align = run < 16 ? run : 16;
    return ((uintptr_t)mask % align) == 0 && (stride_b * msize[mask_dtype]) % align == 0;
}

enum FwdKind { FWD_BCL, FWD_BLC, FWD_GENERIC };
enum UpdKind { UPD_VEC, UPD_GENERIC };

constexpr uint32_t kGenericChunk = 8;   // time steps per thread in the scalar kernel
constexpr int kBlcRows = CANON_BLC_ROWS;   // time steps per wave in the channel-contiguous kernel
constexpr uint64_t kStreamBytes = 64ull << 20;  // above this much traffic, x / out are accessed non-temporally
constexpr int kUpdNB = 2;               // batch rows per lane in the vectorised update when there is plenty of work

struct FwdPlan {
    FwdKind kind;
    int U;
    FwdArgs args;
    uint32_t grid;
};

int plan_fwd(const canon_conv1d_fwd_params *p, FwdPlan *plan)
{
    if (!p) return fail(CANON_ERR_INVALID_ARGUMENT, "params is NULL");
    if (p->struct_size != sizeof(canon_conv1d_fwd_params))
        return fail(CANON_ERR_INVALID_ARGUMENT, "struct_size %u does not match this library's canon_conv1d_fwd_params (%zu)",
                    p->struct_size, sizeof(canon_conv1d_fwd_params));
    if (!valid_dtype(p->x_dtype) || !valid_dtype(p->w_dtype))
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown x_dtype %d or w_dtype %d", p->x_dtype, p->w_dtype);
    if (p->width < CANON_CONV1D_MIN_WIDTH || p->width > CANON_CONV1D_MAX_WIDTH)
        return fail(CANON_ERR_UNSUPPORTED, "width %d not supported (only widths 2..4)", p->width);
    if (p->activation != CANON_ACT_NONE && p->activation != CANON_ACT_SILU)
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown activation %d", p->activation);
    if (p->residual_mode < CANON_RESIDUAL_NONE || p->residual_mode > CANON_RESIDUAL_UNMASKED)
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown residual_mode %d", p->residual_mode);
    if (p->round_mode != CANON_ROUND_FUSED && p->round_mode != CANON_ROUND_EAGER)
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown round_mode %d", p->round_mode);
    if (p->batch < 0 || p->channels < 0 || p->seqlen < 0)
        return fail(CANON_ERR_INVALID_ARGUMENT, "negative size (batch %lld, channels %lld, seqlen %lld)",
                    (long long)p->batch, (long long)p->channels, (long long)p->seqlen);
    if (p->batch >= (1ll << 31) || p->channels >= (1ll << 31) || p->seqlen >= (1ll << 31) ||
        p->batch * p->channels >= (1ll << 31))
        return fail(CANON_ERR_UNSUPPORTED, "batch*channels and seqlen must each be below 2^31");
    const bool empty = p->batch == 0 || p->channels == 0 || p->seqlen == 0;
    if (!empty) {
        if (!p->x || !p->out || !p->weight) return fail(CANON_ERR_INVALID_ARGUMENT, "x, out and weight must not be NULL");
        if (p->x == p->out) return fail(CANON_ERR_INVALID_ARGUMENT, "out must not alias x");
    }
    if (p->mask && !valid_mask_dtype(p->mask_dtype))
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown mask_dtype %d", p->mask_dtype);
    if (p->initial_state && p->initial_len < p->width - 1)
        return fail(CANON_ERR_INVALID_ARGUMENT, "initial_len %d is shorter than width-1 = %d", p->initial_len, p->width - 1);
    if (p->final_state && p->final_len < 1)
        return fail(CANON_ERR_INVALID_ARGUMENT, "final_len %d must be at least 1", p->final_len);
    if (p->final_state && p->final_len > 64)
        return fail(CANON_ERR_UNSUPPORTED, "final_len %d above 64 is not supported", p->final_len);
    if (p->seq_idx && (p->initial_state || p->final_state))
        return fail(CANON_ERR_INVALID_ARGUMENT, "seq_idx excludes initial_state and final_state");
    if (p->seq_idx && ((uintptr_t)p->seq_idx & 3u))
        return fail(CANON_ERR_INVALID_ARGUMENT, "seq_idx must be 4-byte aligned");

    FwdArgs &a = plan->args;
    memset(&a, 0, sizeof(a));
    a.x = (const char *)p->x; a.out = (char *)p->out;
    a.weight = p->weight; a.bias = p->bias; a.mask = p->mask;
    a.init = p->initial_state; a.fin = p->final_state;
    a.seq = p->seq_idx; a.q_sb = p->seq_stride_b; a.q_sl = p->seq_stride_l;
    a.x_sb = p->x_stride_b; a.x_sc = p->x_stride_c; a.x_sl = p->x_stride_l;
    a.o_sb = p->out_stride_b; a.o_sc = p->out_stride_c; a.o_sl = p->out_stride_l;
    a.w_sc = p->w_stride_c; a.w_sk = p->w_stride_k;
    a.m_sb = p->mask_stride_b; a.m_sl = p->mask_stride_l;
    a.i_sb = p->init_stride_b; a.i_sc = p->init_stride_c; a.i_ss = p->init_stride_s;
    a.f_sb = p->final_stride_b; a.f_sc = p->final_stride_c; a.f_ss = p->final_stride_s;
    a.B = (uint32_t)p->batch; a.C = (uint32_t)p->channels; a.L = (uint32_t)p->seqlen;
    a.W = p->width; a.w_dtype = p->w_dtype; a.mask_dtype = p->mask_dtype;
    a.act = p->activation; a.res_mode = p->residual_mode; a.eager = p->round_mode;
    a.S_in = p->initial_state ? p->initial_len : 0;
    a.S_out = p->final_state ? p->final_len : 0;
    a.w_vec = p->width == 4 && p->w_stride_k == 1 && p->w_stride_c == 4 && aligned16(p->weight);
    a.b_vec = p->bias && aligned16(p->bias);
    a.m_vec = mask_run_aligned(p->mask, p->mask_dtype, p->mask_stride_b, p->mask_stride_l, p->x_dtype);
    a.b_pair = p->bias && ((uintptr_t)p->bias & 3u) == 0 && (p->w_dtype == CANON_DTYPE_F32 || p->channels % 2 == 0);
    plan->U = 1;
    plan->grid = 0;
    plan->kind = FWD_GENERIC;
    if (empty) return CANON_OK;

    const int E = 16 / elem_bytes(p->x_dtype);
    const uint64_t rows = (uint64_t)a.B * a.C;
    a.nt = 2 * rows * a.L * elem_bytes(p->x_dtype) >= kStreamBytes;
    const bool fused = p->round_mode == CANON_ROUND_FUSED;
    const bool ptr_ok = aligned16(p->x) && aligned16(p->out);
    // packed sequences: the channel-contiguous kernel has a variant (the index is uniform per time row);
    // time-contiguous rows take the strided kernel
    const bool bcl_ok = !p->seq_idx && fused && ptr_ok && a.x_sl == 1 && a.o_sl == 1 && a.L % E == 0 &&
                        a.x_sb % E == 0 && a.x_sc % E == 0 && a.o_sb % E == 0 && a.o_sc % E == 0 &&
                        a.L / E >= 16;
    const uint32_t EB = kBlcVecBytes / elem_bytes(p->x_dtype);   // channels per lane of the channel-contiguous kernel
    const bool ptr8_ok = (((uintptr_t)p->x | (uintptr_t)p->out) & (kBlcVecBytes - 1)) == 0;
    const bool blc_ok = fused && ptr8_ok && a.x_sc == 1 && a.o_sc == 1 && a.C % EB == 0 &&
                        a.x_sb % EB == 0 && a.x_sl % EB == 0 && a.o_sb % EB == 0 && a.o_sl % EB == 0 &&
                        a.x_sl != 1;

    if (bcl_ok) {
        const uint32_t nvec = a.L / E;
        // vectors per lane: as many as keep >= 2048 waves in flight, at most 4
        int U = 1;
        for (int cand = 2; cand <= 4; cand *= 2) {
            const uint64_t nseg = (nvec + 64u * cand - 1) / (64u * cand);
            if (nvec >= 64u * cand && rows * nseg >= 2048) U = cand;
        }
        const uint64_t nseg = (nvec + 64u * U - 1) / (64u * U);
        const uint64_t ntasks = rows * nseg;
        if (ntasks < (1ull << 31)) {
            plan->kind = FWD_BCL;
            plan->U = U;
            a.nvec = nvec; a.nseg = (uint32_t)nseg; a.ntasks = (uint32_t)ntasks;
            a.div_nseg = make_fastdiv(a.nseg); a.div_C = make_fastdiv(a.C);
            a.nblocks = (uint32_t)((ntasks + 3) / 4);
            plan->grid = a.nblocks;
            return CANON_OK;
        }
    }
    if (blc_ok) {
        const uint32_t nvec = a.C / EB;
        const uint32_t nct = (nvec + 63) / 64;                                   // channel tiles per row
        const uint32_t ntt = (a.L + kBlcWaves * kBlcRows - 1) / (kBlcWaves * kBlcRows);   // time tiles per sequence
        const uint64_t nblocks = (uint64_t)a.B * ntt * nct;
        if (nblocks < (1ull << 31) - 8) {
            plan->kind = FWD_BLC;
            a.nvec = nvec; a.nct = nct; a.ntt = ntt; a.ntasks = (uint32_t)nblocks;
            a.div_nct = make_fastdiv(nct); a.div_ntt = make_fastdiv(ntt);
            a.nblocks = (uint32_t)nblocks;
            plan->grid = a.nblocks;
            return CANON_OK;
        }
    }
    {
        const uint32_t nseg = (a.L + kGenericChunk - 1) / kGenericChunk;
        const uint64_t nthreads = rows * nseg;
        if (nthreads >= (1ull << 32))
            return fail(CANON_ERR_UNSUPPORTED, "problem too large for the strided kernel (%llu threads)",
                        (unsigned long long)nthreads);
        plan->kind = FWD_GENERIC;
        a.nseg = nseg; a.chunk = kGenericChunk; a.ntasks = (uint32_t)nthreads;
        a.nblocks = (uint32_t)((nthreads + 255) / 256);
        plan->grid = a.nblocks;
    }
    return CANON_OK;
}

template <int DT, int W, bool MASK, bool NT> void launch_bcl(const FwdPlan &pl, hipStream_t s)
{
    const dim3 g(pl.grid), b(256);
    switch (pl.U) {
    case 4: hipLaunchKernelGGL((canon_fwd_bcl_kernel<DT, W, 4, MASK, NT>), g, b, 0, s, pl.args); break;
    case 2: hipLaunchKernelGGL((canon_fwd_bcl_kernel<DT, W, 2, MASK, NT>), g, b, 0, s, pl.args); break;
    default: hipLaunchKernelGGL((canon_fwd_bcl_kernel<DT, W, 1, MASK, NT>), g, b, 0, s, pl.args); break;
    }
}

template <int DT, int W, bool MASK, bool NT> void launch_fwd_vec(const FwdPlan &pl, hipStream_t s)
{
    if (pl.kind == FWD_BCL) launch_bcl<DT, W, MASK, NT>(pl, s);
    else hipLaunchKernelGGL((canon_fwd_blc_kernel<DT, W, kBlcRows, MASK, NT>), dim3(pl.grid), dim3(256), 0, s, pl.args);
}

template <int DT, int W> void launch_fwd_w(const FwdPlan &pl, hipStream_t s)
{
    const bool mask = pl.args.mask != nullptr;
    if (pl.args.seq) {   // only the channel-contiguous kernel is planned with seq_idx
        if (mask) hipLaunchKernelGGL((canon_fwd_blc_seq_kernel<DT, W, kBlcRows, true>), dim3(pl.grid), dim3(256), 0, s, pl.args);
        else hipLaunchKernelGGL((canon_fwd_blc_seq_kernel<DT, W, kBlcRows, false>), dim3(pl.grid), dim3(256), 0, s, pl.args);
        return;
    }
    // the streaming (non-temporal) variants exist for width 4 only
    if (W == 4 && pl.args.nt) {
        if (mask) launch_fwd_vec<DT, W, true, W == 4>(pl, s);
        else launch_fwd_vec<DT, W, false, W == 4>(pl, s);
    } else {
        if (mask) launch_fwd_vec<DT, W, true, false>(pl, s);
        else launch_fwd_vec<DT, W, false, false>(pl, s);
    }
}

template <int DT> void launch_fwd(const FwdPlan &pl, hipStream_t s)
{
    if (pl.kind == FWD_GENERIC) {
        hipLaunchKernelGGL((canon_fwd_generic_kernel<DT>), dim3(pl.grid), dim3(256), 0, s, pl.args);
        return;
    }
    switch (pl.args.W) {
    case 2: launch_fwd_w<DT, 2>(pl, s); break;
    case 3: launch_fwd_w<DT, 3>(pl, s); break;
    default: launch_fwd_w<DT, 4>(pl, s); break;
    }
}

struct UpdPlan {
    UpdKind kind;
    UpdArgs args;
    uint32_t grid;
};

int plan_update(const canon_conv1d_update_params *p, UpdPlan *plan)
{
    if (!p) return fail(CANON_ERR_INVALID_ARGUMENT, "params is NULL");
    if (p->struct_size != sizeof(canon_conv1d_update_params))
        return fail(CANON_ERR_INVALID_ARGUMENT, "struct_size %u does not match this library's canon_conv1d_update_params (%zu)",
                    p->struct_size, sizeof(canon_conv1d_update_params));
    if (!valid_dtype(p->x_dtype) || !valid_dtype(p->w_dtype))
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown x_dtype %d or w_dtype %d", p->x_dtype, p->w_dtype);
    if (p->width < CANON_CONV1D_MIN_WIDTH || p->width > CANON_CONV1D_MAX_WIDTH)
        return fail(CANON_ERR_UNSUPPORTED, "width %d not supported (only widths 2..4)", p->width);
    if (p->activation != CANON_ACT_NONE && p->activation != CANON_ACT_SILU)
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown activation %d", p->activation);
    if (p->residual_mode < CANON_RESIDUAL_NONE || p->residual_mode > CANON_RESIDUAL_UNMASKED)
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown residual_mode %d", p->residual_mode);
    if (p->round_mode != CANON_ROUND_FUSED && p->round_mode != CANON_ROUND_EAGER)
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown round_mode %d", p->round_mode);
    if (p->cache_seqlens) return fail(CANON_ERR_UNSUPPORTED, "cache_seqlens (circular conv_state) is not supported");
    if (p->conv_state_indices) return fail(CANON_ERR_UNSUPPORTED, "conv_state_indices is not supported");
    if (p->batch < 0 || p->channels < 0)
        return fail(CANON_ERR_INVALID_ARGUMENT, "negative size (batch %lld, channels %lld)", (long long)p->batch, (long long)p->channels);
    if (p->batch >= (1ll << 31) || p->channels >= (1ll << 31) || p->batch * p->channels >= (1ll << 31))
        return fail(CANON_ERR_UNSUPPORTED, "batch*channels must be below 2^31");
    if (p->state_len < 1 || p->state_len < p->width - 1)
        return fail(CANON_ERR_INVALID_ARGUMENT, "state_len %d is shorter than width-1 = %d", p->state_len, p->width - 1);
    const bool empty = p->batch == 0 || p->channels == 0;
    if (!empty && (!p->x || !p->out || !p->conv_state || !p->weight))
        return fail(CANON_ERR_INVALID_ARGUMENT, "x, out, conv_state and weight must not be NULL");
    if (p->token_mask && !valid_mask_dtype(p->mask_dtype))
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown mask_dtype %d", p->mask_dtype);

    UpdArgs &a = plan->args;
    memset(&a, 0, sizeof(a));
    a.x = (const char *)p->x; a.out = (char *)p->out; a.state = (char *)p->conv_state;
    a.weight = p->weight; a.bias = p->bias; a.tmask = p->token_mask;
    a.x_sb = p->x_stride_b; a.x_sc = p->x_stride_c; a.o_sb = p->out_stride_b; a.o_sc = p->out_stride_c;
    a.s_sb = p->state_stride_b; a.s_sc = p->state_stride_c; a.s_ss = p->state_stride_s;
    a.w_sc = p->w_stride_c; a.w_sk = p->w_stride_k; a.m_sb = p->mask_stride_b;
    a.B = (uint32_t)p->batch; a.C = (uint32_t)p->channels;
    a.W = p->width; a.S = p->state_len; a.w_dtype = p->w_dtype; a.mask_dtype = p->mask_dtype;
    a.act = p->activation; a.res_mode = p->residual_mode; a.eager = p->round_mode;
    a.w_vec = p->width == 4 && p->w_stride_k == 1 && p->w_stride_c == 4 && aligned16(p->weight);
    a.b_vec = p->bias && aligned16(p->bias);
    plan->kind = UPD_GENERIC;
    plan->grid = 0;
    if (empty) return CANON_OK;

    const int E = 16 / elem_bytes(p->x_dtype);
    const int S = p->state_len;
    const bool vec_ok = p->round_mode == CANON_ROUND_FUSED && (S == 3 || S == 4 || S == 8) &&
                        aligned16(p->x) && aligned16(p->out) && aligned16(p->conv_state) &&
                        a.x_sc == 1 && a.o_sc == 1 && a.C % E == 0 && a.x_sb % E == 0 && a.o_sb % E == 0 &&
                        a.s_ss == 1 && a.s_sc == S && a.s_sb % E == 0;
    if (vec_ok) {
        plan->kind = UPD_VEC;
        a.nvec = a.C / E;
        // two batch rows per lane halve the tap loads; with little work, more waves matter more
        a.nb = ((uint64_t)a.nvec * a.B / kUpdNB >= 512 * 64) ? kUpdNB : 1;
        a.bgroups = (a.B + a.nb - 1) / a.nb;
        a.nthreads = a.nvec * a.bgroups;
        a.div_nvec = make_fastdiv(a.nvec);
        plan->grid = (a.nthreads + 255) / 256;
    } else {
        a.nthreads = a.B * a.C;
        plan->grid = (a.nthreads + 255) / 256;
    }
    return CANON_OK;
}

template <int DT, int W, int NB> void launch_update_vec_nb(const UpdPlan &pl, hipStream_t s)
{
    const dim3 g(pl.grid), b(256);
    switch (pl.args.S) {
    case 3: hipLaunchKernelGGL((canon_update_vec_kernel<DT, W, 3, NB>), g, b, 0, s, pl.args); break;
    case 4: hipLaunchKernelGGL((canon_update_vec_kernel<DT, W, 4, NB>), g, b, 0, s, pl.args); break;
    default: hipLaunchKernelGGL((canon_update_vec_kernel<DT, W, 8, NB>), g, b, 0, s, pl.args); break;
    }
}

template <int DT, int W> void launch_update_vec_w(const UpdPlan &pl, hipStream_t s)
{
    if (pl.args.nb == kUpdNB) launch_update_vec_nb<DT, W, kUpdNB>(pl, s);
    else launch_update_vec_nb<DT, W, 1>(pl, s);
}

template <int DT> void launch_update(const UpdPlan &pl, hipStream_t s)
{
    if (pl.kind == UPD_GENERIC) {
        hipLaunchKernelGGL((canon_update_generic_kernel<DT>), dim3(pl.grid), dim3(256), 0, s, pl.args);
        return;
    }
    switch (pl.args.W) {
    case 2: launch_update_vec_w<DT, 2>(pl, s); break;
    case 3: launch_update_vec_w<DT, 3>(pl, s); break;
    default: launch_update_vec_w<DT, 4>(pl, s); break;
    }
}

// ---------------------------------------------------------------------------
// channel ranges in separate tensors: one derived problem per part
// ---------------------------------------------------------------------------
const void *advance(const void *p, int64_t elems, int bytes)
{
    return p ? (const void *)((const char *)p + elems * bytes) : nullptr;
}

int check_parts(const canon_conv1d_part *parts, int32_t nparts, int64_t channels)
{
    if (!parts) return fail(CANON_ERR_INVALID_ARGUMENT, "parts is NULL");
    if (nparts < 1 || nparts > kMaxParts)
        return fail(CANON_ERR_INVALID_ARGUMENT, "nparts %d outside 1..%d", nparts, kMaxParts);
    int64_t sum = 0;
    for (int i = 0; i < nparts; ++i) {
        if (parts[i].channels < 0 || parts[i].channels >= (1ll << 31))
            return fail(CANON_ERR_INVALID_ARGUMENT, "part %d has %lld channels", i, (long long)parts[i].channels);
        sum += parts[i].channels;
    }
    if (sum != channels)
        return fail(CANON_ERR_INVALID_ARGUMENT, "the parts hold %lld channels, params.channels is %lld", (long long)sum,
                    (long long)channels);
    return CANON_OK;
}

struct FwdPartsPlan {
    int n;
    bool single;            // one launch over a PartTable
    uint32_t grid;          // of that launch
    FwdPlan part[kMaxParts];
};

int plan_fwd_parts(const canon_conv1d_fwd_params *p, const canon_conv1d_part *parts, int32_t nparts, FwdPartsPlan *pp)
{
    if (!p) return fail(CANON_ERR_INVALID_ARGUMENT, "params is NULL");
    if (p->struct_size != sizeof(canon_conv1d_fwd_params))
        return fail(CANON_ERR_INVALID_ARGUMENT, "struct_size %u does not match this library's canon_conv1d_fwd_params (%zu)",
                    p->struct_size, sizeof(canon_conv1d_fwd_params));
    if (!valid_dtype(p->x_dtype) || !valid_dtype(p->w_dtype))
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown x_dtype %d or w_dtype %d", p->x_dtype, p->w_dtype);
    int rc = check_parts(parts, nparts, p->channels);
    if (rc != CANON_OK) return rc;
    if (p->batch > 0 && p->batch * p->channels >= (1ll << 31))
        return fail(CANON_ERR_UNSUPPORTED, "batch*channels and seqlen must each be below 2^31");
    const int xb = elem_bytes(p->x_dtype), wb = elem_bytes(p->w_dtype);
    pp->n = nparts;
    int64_t c0 = 0;
    uint64_t blocks = 0;
    bool all_blc = true;
    for (int i = 0; i < nparts; ++i) {
        canon_conv1d_fwd_params q = *p;
        q.channels = parts[i].channels;
        q.x = parts[i].x; q.x_stride_b = parts[i].x_stride_b; q.x_stride_c = parts[i].x_stride_c; q.x_stride_l = parts[i].x_stride_l;
        q.out = parts[i].out; q.out_stride_b = parts[i].out_stride_b; q.out_stride_c = parts[i].out_stride_c;
        q.out_stride_l = parts[i].out_stride_l;
        q.weight = advance(p->weight, c0 * p->w_stride_c, wb);
        q.bias = advance(p->bias, c0, wb);
        q.initial_state = advance(p->initial_state, c0 * p->init_stride_c, xb);
        q.final_state = (void *)advance(p->final_state, c0 * p->final_stride_c, xb);
        rc = plan_fwd(&q, &pp->part[i]);
        if (rc != CANON_OK) return rc;
        if (pp->part[i].grid > 0) {
            all_blc = all_blc && pp->part[i].kind == FWD_BLC;
            blocks += pp->part[i].grid;
        }
        c0 += parts[i].channels;
    }
    // whether to stream past the caches is decided on the whole problem
    const bool nt = 2ull * (uint64_t)p->batch * (uint64_t)p->channels * (uint64_t)p->seqlen * xb >= kStreamBytes;
    for (int i = 0; i < nparts; ++i) pp->part[i].args.nt = nt;
    pp->single = nparts > 1 && all_blc && p->width == 4 && !p->seq_idx && blocks > 0 && blocks < (1ull << 31);
    pp->grid = (uint32_t)blocks;
    return CANON_OK;
}

template <int DT, bool MASK, bool NT>
void launch_blc_parts(const PartTable<FwdArgs> &m, uint32_t grid, hipStream_t s)
{
    hipLaunchKernelGGL((canon_fwd_blc_parts_kernel<DT, 4, kBlcRows, MASK, NT>), dim3(grid), dim3(256), 0, s, m);
}

template <int DT> void launch_fwd_parts(const FwdPartsPlan &pp, hipStream_t s)
{
    if (!pp.single) {
        for (int i = 0; i < pp.n; ++i)
            if (pp.part[i].grid > 0) launch_fwd<DT>(pp.part[i], s);
        return;
    }
    PartTable<FwdArgs> m;
    memset(&m, 0, sizeof(m));
    uint32_t first = 0;
    bool mask = false, nt = false;
    for (int i = 0; i < kMaxParts; ++i) {
        m.first_block[i] = i < pp.n ? first : 0xFFFFFFFFu;
        if (i < pp.n) {
            m.part[i] = pp.part[i].args;
            first += pp.part[i].grid;
            mask = pp.part[i].args.mask != nullptr;
            nt = pp.part[i].args.nt != 0;
        }
    }
    if (mask) {
        if (nt) launch_blc_parts<DT, true, true>(m, pp.grid, s);
        else launch_blc_parts<DT, true, false>(m, pp.grid, s);
    } else {
        if (nt) launch_blc_parts<DT, false, true>(m, pp.grid, s);
        else launch_blc_parts<DT, false, false>(m, pp.grid, s);
    }
}

struct UpdPartsPlan {
    int n;
    bool single;
    uint32_t grid;
    UpdPlan part[kMaxParts];
};

int plan_update_parts(const canon_conv1d_update_params *p, const canon_conv1d_part *parts, int32_t nparts, UpdPartsPlan *pp)
{
    if (!p) return fail(CANON_ERR_INVALID_ARGUMENT, "params is NULL");
    if (p->struct_size != sizeof(canon_conv1d_update_params))
        return fail(CANON_ERR_INVALID_ARGUMENT, "struct_size %u does not match this library's canon_conv1d_update_params (%zu)",
                    p->struct_size, sizeof(canon_conv1d_update_params));
    if (!valid_dtype(p->x_dtype) || !valid_dtype(p->w_dtype))
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown x_dtype %d or w_dtype %d", p->x_dtype, p->w_dtype);
    int rc = check_parts(parts, nparts, p->channels);
    if (rc != CANON_OK) return rc;
    if (p->batch > 0 && p->batch * p->channels >= (1ll << 31))
        return fail(CANON_ERR_UNSUPPORTED, "batch*channels must be below 2^31");
    const int xb = elem_bytes(p->x_dtype), wb = elem_bytes(p->w_dtype);
    pp->n = nparts;
    int64_t c0 = 0;
    bool all_vec = true;
    uint64_t nvec_total = 0;
    for (int i = 0; i < nparts; ++i) {
        canon_conv1d_update_params q = *p;
        q.channels = parts[i].channels;
        q.x = parts[i].x; q.x_stride_b = parts[i].x_stride_b; q.x_stride_c = parts[i].x_stride_c;
        q.out = parts[i].out; q.out_stride_b = parts[i].out_stride_b; q.out_stride_c = parts[i].out_stride_c;
        q.conv_state = (void *)advance(p->conv_state, c0 * p->state_stride_c, xb);
        q.weight = advance(p->weight, c0 * p->w_stride_c, wb);
        q.bias = advance(p->bias, c0, wb);
        rc = plan_update(&q, &pp->part[i]);
        if (rc != CANON_OK) return rc;
        if (pp->part[i].grid > 0) {
            all_vec = all_vec && pp->part[i].kind == UPD_VEC;
            nvec_total += pp->part[i].args.nvec;
        }
        c0 += parts[i].channels;
    }
    pp->single = nparts > 1 && all_vec && p->width == 4 && nvec_total > 0;
    pp->grid = 0;
    if (pp->single) {
        // batch rows per lane chosen on the whole token, the same for every part
        const uint32_t nb = (nvec_total * (uint64_t)p->batch / kUpdNB >= 512 * 64) ? kUpdNB : 1;
        uint64_t blocks = 0;
        for (int i = 0; i < nparts; ++i) {
            UpdPlan &u = pp->part[i];
            if (u.grid == 0) continue;
            u.args.nb = nb;
            u.args.bgroups = (u.args.B + nb - 1) / nb;
            u.args.nthreads = u.args.nvec * u.args.bgroups;
            u.grid = (u.args.nthreads + 255) / 256;
            blocks += u.grid;
        }
        pp->grid = (uint32_t)blocks;
    }
    return CANON_OK;
}

template <int DT, int NB> void launch_update_parts_nb(const PartTable<UpdArgs> &m, int S, uint32_t grid, hipStream_t s)
{
    const dim3 g(grid), b(256);
    switch (S) {
    case 3: hipLaunchKernelGGL((canon_update_vec_parts_kernel<DT, 4, 3, NB>), g, b, 0, s, m); break;
    case 4: hipLaunchKernelGGL((canon_update_vec_parts_kernel<DT, 4, 4, NB>), g, b, 0, s, m); break;
    default: hipLaunchKernelGGL((canon_update_vec_parts_kernel<DT, 4, 8, NB>), g, b, 0, s, m); break;
    }
}

template <int DT> void launch_update_parts(const UpdPartsPlan &pp, hipStream_t s)
{
    if (!pp.single) {
        for (int i = 0; i < pp.n; ++i)
            if (pp.part[i].grid > 0) launch_update<DT>(pp.part[i], s);
        return;
    }
    PartTable<UpdArgs> m;
    memset(&m, 0, sizeof(m));
    uint32_t first = 0, nb = 1;
    int S = 0;
    for (int i = 0; i < kMaxParts; ++i) {
        m.first_block[i] = i < pp.n ? first : 0xFFFFFFFFu;
        if (i < pp.n) {
            m.part[i] = pp.part[i].args;
            first += pp.part[i].grid;
            if (pp.part[i].grid > 0) {
                nb = pp.part[i].args.nb;
                S = pp.part[i].args.S;
            }
        }
    }
    if (nb == kUpdNB) launch_update_parts_nb<DT, kUpdNB>(m, S, pp.grid, s);
    else launch_update_parts_nb<DT, 1>(m, S, pp.grid, s);
}

// ---------------------------------------------------------------------------
// backward: planning and launch
// ---------------------------------------------------------------------------
enum BwdKind { BWD_BLC_VEC, BWD_BCL_VEC, BWD_GENERIC };
constexpr int kBwdRows = 4;   // rows fetched ahead per lane in the backward walk
constexpr int kBwdHalfBlocksPerCU = 3;   // grid target of the channel-contiguous backward, in half blocks per CU

struct BwdPlan {
    BwdKind kind;
    int U;
    BwdArgs args;
    uint32_t grid;
    int64_t workspace_bytes;
};

int plan_bwd(const canon_conv1d_bwd_params *p, BwdPlan *plan, bool check_pointers)
{
    if (!p) return fail(CANON_ERR_INVALID_ARGUMENT, "params is NULL");
    if (p->struct_size != sizeof(canon_conv1d_bwd_params))
        return fail(CANON_ERR_INVALID_ARGUMENT, "struct_size %u does not match this library's canon_conv1d_bwd_params (%zu)",
                    p->struct_size, sizeof(canon_conv1d_bwd_params));
    if (!valid_dtype(p->x_dtype) || !valid_dtype(p->w_dtype))
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown x_dtype %d or w_dtype %d", p->x_dtype, p->w_dtype);
    if (p->width < CANON_CONV1D_MIN_WIDTH || p->width > CANON_CONV1D_MAX_WIDTH)
        return fail(CANON_ERR_UNSUPPORTED, "width %d not supported (only widths 2..4)", p->width);
    if (p->activation != CANON_ACT_NONE && p->activation != CANON_ACT_SILU)
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown activation %d", p->activation);
    if (p->residual_mode < CANON_RESIDUAL_NONE || p->residual_mode > CANON_RESIDUAL_UNMASKED)
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown residual_mode %d", p->residual_mode);
    if (p->batch < 0 || p->channels < 0 || p->seqlen < 0)
        return fail(CANON_ERR_INVALID_ARGUMENT, "negative size (batch %lld, channels %lld, seqlen %lld)",
                    (long long)p->batch, (long long)p->channels, (long long)p->seqlen);
    if (p->batch >= (1ll << 31) || p->channels >= (1ll << 31) || p->seqlen >= (1ll << 31) ||
        p->batch * p->channels >= (1ll << 31))
        return fail(CANON_ERR_UNSUPPORTED, "batch*channels and seqlen must each be below 2^31");
    if (p->mask && !valid_mask_dtype(p->mask_dtype))
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown mask_dtype %d", p->mask_dtype);
    const bool empty = p->batch == 0 || p->channels == 0 || p->seqlen == 0;
    if (check_pointers) {
        if (p->channels > 0 && (!p->weight || !p->dweight))
            return fail(CANON_ERR_INVALID_ARGUMENT, "weight and dweight must not be NULL");
        if (!empty && (!p->x || !p->dout || !p->dx))
            return fail(CANON_ERR_INVALID_ARGUMENT, "x, dout and dx must not be NULL");
        if (!empty && (p->dx == p->x || p->dx == p->dout))
            return fail(CANON_ERR_INVALID_ARGUMENT, "dx must not alias x or dout");
    }

    BwdArgs &a = plan->args;
    memset(&a, 0, sizeof(a));
    a.x = (const char *)p->x; a.dy = (const char *)p->dout; a.dx = (char *)p->dx;
    a.weight = p->weight; a.bias = p->bias; a.mask = p->mask;
    a.partial = (float *)p->workspace; a.dweight = p->dweight; a.dbias = p->dbias;
    a.x_sb = p->x_stride_b; a.x_sc = p->x_stride_c; a.x_sl = p->x_stride_l;
    a.g_sb = p->dout_stride_b; a.g_sc = p->dout_stride_c; a.g_sl = p->dout_stride_l;
    a.d_sb = p->dx_stride_b; a.d_sc = p->dx_stride_c; a.d_sl = p->dx_stride_l;
    a.w_sc = p->w_stride_c; a.w_sk = p->w_stride_k;
    a.m_sb = p->mask_stride_b; a.m_sl = p->mask_stride_l;
    a.B = (uint32_t)p->batch; a.C = (uint32_t)p->channels; a.L = (uint32_t)p->seqlen;
    a.W = p->width; a.w_dtype = p->w_dtype; a.mask_dtype = p->mask_dtype;
    a.act = p->activation; a.res_mode = p->residual_mode;
    a.w_vec = p->width == 4 && p->w_stride_k == 1 && p->w_stride_c == 4 && aligned16(p->weight);
    a.b_vec = p->bias && aligned16(p->bias);
    plan->kind = BWD_GENERIC;
    plan->U = 1;
    plan->grid = 0;
    plan->workspace_bytes = 0;
    if (empty) return CANON_OK;   // the caller's dweight/dbias are zero filled by canon_conv1d_bwd

    const int E = 16 / elem_bytes(p->x_dtype);
    a.b_pair = p->bias && ((uintptr_t)p->bias & 3u) == 0 && (p->w_dtype == CANON_DTYPE_F32 || p->channels % 2 == 0);
    a.m_vec = mask_run_aligned(p->mask, p->mask_dtype, p->mask_stride_b, p->mask_stride_l, p->x_dtype);
    const bool ptrs16 = !check_pointers || (aligned16(p->x) && aligned16(p->dout) && aligned16(p->dx));
    const bool rows = ptrs16 && a.x_sl == 1 && a.g_sl == 1 && a.d_sl == 1 && a.L % E == 0 && a.L / E >= 16 &&
                      a.x_sb % E == 0 && a.x_sc % E == 0 && a.g_sb % E == 0 && a.g_sc % E == 0 &&
                      a.d_sb % E == 0 && a.d_sc % E == 0;
    if (rows) {
        const uint32_t nvec = a.L / E;
        const uint64_t nrows = (uint64_t)a.B * a.C;
        int U = 1;
        for (int cand = 2; cand <= 4; cand *= 2) {
            const uint64_t nseg = (nvec + 64u * cand - 1) / (64u * cand);
            if (nvec >= 64u * cand && nrows * nseg >= 2048) U = cand;
        }
        const uint64_t nseg = (nvec + 64u * U - 1) / (64u * U);
        const uint64_t ntasks = nrows * nseg;
        if (ntasks < (1ull << 31)) {
            plan->kind = BWD_BCL_VEC;
            plan->U = U;
            // field use in this kernel family: nthreads = wave tasks, nchunk = segments per row
            a.nvec = nvec; a.nchunk = (uint32_t)nseg; a.nthreads = (uint32_t)ntasks;
            a.nsets = a.B * a.nchunk;
            a.div_nchunk = make_fastdiv(a.nchunk); a.div_nvec = make_fastdiv(a.C);
            plan->grid = (uint32_t)((ntasks + 3) / 4);
            plan->workspace_bytes = (int64_t)a.nsets * a.C * 5 * (int64_t)sizeof(float);
            if (check_pointers && (!p->workspace || !aligned16(p->workspace) || p->workspace_bytes < plan->workspace_bytes))
                return fail(CANON_ERR_INVALID_ARGUMENT, "workspace must be 16-byte aligned and at least %lld bytes (got %lld)",
                            (long long)plan->workspace_bytes, (long long)p->workspace_bytes);
            return CANON_OK;
        }
    }
    // channel-contiguous tensors: 8-byte groups of channels per lane
    const int E8 = 8 / elem_bytes(p->x_dtype);
    const bool ptrs8 = !check_pointers || ((((uintptr_t)p->x | (uintptr_t)p->dout | (uintptr_t)p->dx) & 7u) == 0);
    const bool vec = a.x_sc == 1 && a.g_sc == 1 && a.d_sc == 1 && a.C % E8 == 0 && a.x_sl != 1 &&
                     a.x_sb % E8 == 0 && a.x_sl % E8 == 0 && a.g_sb % E8 == 0 && a.g_sl % E8 == 0 &&
                     a.d_sb % E8 == 0 && a.d_sl % E8 == 0 && ptrs8;
    if (vec) {
        const uint32_t tile = kBwdSlab * kBwdWaves;
        const uint32_t nvec = a.C / E8;
        const uint32_t nct = (nvec + 63) / 64;
        // time steps per block: as long as possible (few partial sets to write and to add up, taps and
        // chunk-end work amortised) while the grid still has one and a half blocks per CU
        uint32_t chunk = tile;
        for (uint32_t cand = 2 * tile; cand <= 32 * tile; cand *= 2) {
            const uint64_t blocks = (uint64_t)a.B * ((a.L + cand - 1) / cand) * nct;
            if (2 * blocks >= 256ull * kBwdHalfBlocksPerCU) chunk = cand;
        }
        const uint32_t nchunk = (a.L + chunk - 1) / chunk;
        const uint64_t blocks = (uint64_t)a.B * nchunk * nct;
        if (blocks < (1ull << 31)) {
            plan->kind = BWD_BLC_VEC;
            a.nvec = nvec; a.nct = nct; a.chunk = chunk; a.nchunk = nchunk;
            a.nsets = a.B * nchunk;
            a.div_nct = make_fastdiv(nct); a.div_nchunk = make_fastdiv(nchunk);
            plan->grid = (uint32_t)blocks;
            plan->workspace_bytes = (int64_t)a.nsets * a.C * 5 * (int64_t)sizeof(float);
            if (check_pointers && (!p->workspace || !aligned16(p->workspace) || p->workspace_bytes < plan->workspace_bytes))
                return fail(CANON_ERR_INVALID_ARGUMENT, "workspace must be 16-byte aligned and at least %lld bytes (got %lld)",
                            (long long)plan->workspace_bytes, (long long)p->workspace_bytes);
            return CANON_OK;
        }
    }
    plan->kind = BWD_GENERIC;
    a.nvec = a.C;
    // time steps per lane: about 8 waves per CU, a multiple of the look-ahead, and few enough
    // partial sets that the scratch stays below ~16 MB
    const uint64_t lanes_per_step = (uint64_t)a.B * a.nvec;
    uint64_t want_chunks = (256ull * 8 * 64 + lanes_per_step - 1) / lanes_per_step;
    const uint64_t max_sets = (16ull << 20) / ((uint64_t)a.C * 20) + 1;
    if ((uint64_t)a.B * want_chunks > max_sets) want_chunks = max_sets / a.B;
    if (want_chunks < 1) want_chunks = 1;
    uint32_t chunk = (uint32_t)((a.L + want_chunks - 1) / want_chunks);
    chunk = ((chunk + kBwdRows - 1) / kBwdRows) * kBwdRows;
    if (chunk < 4 * kBwdRows) chunk = 4 * kBwdRows;
    a.chunk = chunk;
    a.nchunk = (a.L + chunk - 1) / chunk;
    const uint64_t nthreads = lanes_per_step * a.nchunk;
    if (nthreads >= (1ull << 32)) return fail(CANON_ERR_UNSUPPORTED, "problem too large for the backward kernel");
    a.nthreads = (uint32_t)nthreads;
    a.nsets = a.B * a.nchunk;
    a.div_nvec = make_fastdiv(a.nvec);
    a.div_nchunk = make_fastdiv(a.nchunk);
    plan->grid = (uint32_t)((nthreads + 255) / 256);
    plan->workspace_bytes = (int64_t)a.nsets * a.C * 5 * (int64_t)sizeof(float);
    if (check_pointers) {
        if (!p->workspace || !aligned16(p->workspace) || p->workspace_bytes < plan->workspace_bytes)
            return fail(CANON_ERR_INVALID_ARGUMENT, "workspace must be 16-byte aligned and at least %lld bytes (got %lld)",
                        (long long)plan->workspace_bytes, (long long)p->workspace_bytes);
    }
    return CANON_OK;
}

template <int DT, int W, bool MASK> void launch_bwd_m(const BwdPlan &pl, hipStream_t s)
{
    const dim3 g(pl.grid), b(256);
    if (pl.kind == BWD_BCL_VEC) {
        switch (pl.U) {
        case 4: hipLaunchKernelGGL((canon_bwd_bcl_kernel<DT, W, 4, MASK>), g, b, 0, s, pl.args); break;
        case 2: hipLaunchKernelGGL((canon_bwd_bcl_kernel<DT, W, 2, MASK>), g, b, 0, s, pl.args); break;
        default: hipLaunchKernelGGL((canon_bwd_bcl_kernel<DT, W, 1, MASK>), g, b, 0, s, pl.args); break;
        }
    } else if (pl.kind == BWD_BLC_VEC)
    {
        if (pl.args.act) hipLaunchKernelGGL((canon_bwd_blc_kernel<DT, W, MASK, true>), g, b, 0, s, pl.args);
        else hipLaunchKernelGGL((canon_bwd_blc_kernel<DT, W, MASK, false>), g, b, 0, s, pl.args);
    }
    else
        hipLaunchKernelGGL((canon_bwd_walk_kernel<DT, W, 1, false, MASK, kBwdRows>), g, b, 0, s, pl.args);
}

template <int DT> void launch_bwd(const BwdPlan &pl, hipStream_t s)
{
    const bool m = pl.args.mask != nullptr;
    switch (pl.args.W) {
    case 2: m ? launch_bwd_m<DT, 2, true>(pl, s) : launch_bwd_m<DT, 2, false>(pl, s); break;
    case 3: m ? launch_bwd_m<DT, 3, true>(pl, s) : launch_bwd_m<DT, 3, false>(pl, s); break;
    default: m ? launch_bwd_m<DT, 4, true>(pl, s) : launch_bwd_m<DT, 4, false>(pl, s); break;
    }
}

int check_launch(const char *what)
{
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(CANON_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return CANON_OK;
}

}  // namespace

extern "C" {

int canon_conv1d_abi_version(void) { return CANON_CONV1D_ABI_VERSION; }

const char *canon_conv1d_last_error(void) { return g_err; }

int canon_conv1d_fwd(const canon_conv1d_fwd_params *p, void *stream)
{
    FwdPlan pl;
    const int rc = plan_fwd(p, &pl);
    if (rc != CANON_OK) return rc;
    if (pl.grid == 0) return CANON_OK;
    hipStream_t s = (hipStream_t)stream;
    switch (p->x_dtype) {
    case CANON_DTYPE_F32: launch_fwd<CANON_DTYPE_F32>(pl, s); break;
    case CANON_DTYPE_BF16: launch_fwd<CANON_DTYPE_BF16>(pl, s); break;
    default: launch_fwd<CANON_DTYPE_F16>(pl, s); break;
    }
    return check_launch("canon_conv1d_fwd");
}

int canon_conv1d_update(const canon_conv1d_update_params *p, void *stream)
{
    UpdPlan pl;
    const int rc = plan_update(p, &pl);
    if (rc != CANON_OK) return rc;
    if (pl.grid == 0) return CANON_OK;
    hipStream_t s = (hipStream_t)stream;
    switch (p->x_dtype) {
    case CANON_DTYPE_F32: launch_update<CANON_DTYPE_F32>(pl, s); break;
    case CANON_DTYPE_BF16: launch_update<CANON_DTYPE_BF16>(pl, s); break;
    default: launch_update<CANON_DTYPE_F16>(pl, s); break;
    }
    return check_launch("canon_conv1d_update");
}

int canon_conv1d_bwd(const canon_conv1d_bwd_params *p, void *stream)
{
    BwdPlan pl;
    const int rc = plan_bwd(p, &pl, true);
    if (rc != CANON_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    if (pl.grid == 0) {
        // nothing to sum: the gradients of the parameters are zero
        // (a fill kernel rather than a memset, so that the call can be captured into a HIP graph)
        if (p->channels > 0) {
            const uint32_t nw = (uint32_t)(p->channels * p->width), nc = (uint32_t)p->channels;
            hipLaunchKernelGGL(canon_zero_kernel, dim3((nw + 255) / 256), dim3(256), 0, s, p->dweight, nw);
            if (p->dbias) hipLaunchKernelGGL(canon_zero_kernel, dim3((nc + 255) / 256), dim3(256), 0, s, p->dbias, nc);
            return check_launch("canon_conv1d_bwd");
        }
        return CANON_OK;
    }
    switch (p->x_dtype) {
    case CANON_DTYPE_F32: launch_bwd<CANON_DTYPE_F32>(pl, s); break;
    case CANON_DTYPE_BF16: launch_bwd<CANON_DTYPE_BF16>(pl, s); break;
    default: launch_bwd<CANON_DTYPE_F16>(pl, s); break;
    }
    hipLaunchKernelGGL(canon_bwd_reduce_kernel, dim3((pl.args.C * 5u + 31u) / 32u), dim3(256), 0, s,
                       pl.args.partial, pl.args.dweight, pl.args.dbias, pl.args.C, pl.args.nsets, pl.args.W);
    return check_launch("canon_conv1d_bwd");
}

int64_t canon_conv1d_bwd_workspace_bytes(const canon_conv1d_bwd_params *p)
{
    BwdPlan pl;
    if (plan_bwd(p, &pl, false) != CANON_OK) return -1;
    return pl.workspace_bytes;
}

const char *canon_conv1d_bwd_plan(const canon_conv1d_bwd_params *p)
{
    BwdPlan pl;
    if (plan_bwd(p, &pl, false) != CANON_OK) return nullptr;
    return pl.kind == BWD_BLC_VEC ? "bwd_blc_vec" : pl.kind == BWD_BCL_VEC ? "bwd_bcl_vec" : "bwd_generic";
}

const char *canon_conv1d_fwd_plan(const canon_conv1d_fwd_params *p)
{
    FwdPlan pl;
    if (plan_fwd(p, &pl) != CANON_OK) return nullptr;
    if (pl.kind == FWD_BLC && pl.args.seq) return "blc_vec_seq";
    return pl.kind == FWD_BCL ? "bcl_vec" : pl.kind == FWD_BLC ? "blc_vec" : "generic";
}

const char *canon_conv1d_update_plan(const canon_conv1d_update_params *p)
{
    UpdPlan pl;
    if (plan_update(p, &pl) != CANON_OK) return nullptr;
    return pl.kind == UPD_VEC ? "update_vec" : "update_generic";
}

int canon_conv1d_fwd_parts(const canon_conv1d_fwd_params *p, const canon_conv1d_part *parts, int32_t nparts, void *stream)
{
    FwdPartsPlan pp;
    const int rc = plan_fwd_parts(p, parts, nparts, &pp);
    if (rc != CANON_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    switch (p->x_dtype) {
    case CANON_DTYPE_F32: launch_fwd_parts<CANON_DTYPE_F32>(pp, s); break;
    case CANON_DTYPE_BF16: launch_fwd_parts<CANON_DTYPE_BF16>(pp, s); break;
    default: launch_fwd_parts<CANON_DTYPE_F16>(pp, s); break;
    }
    return check_launch("canon_conv1d_fwd_parts");
}

int canon_conv1d_update_parts(const canon_conv1d_update_params *p, const canon_conv1d_part *parts, int32_t nparts,
                              void *stream)
{
    UpdPartsPlan pp;
    const int rc = plan_update_parts(p, parts, nparts, &pp);
    if (rc != CANON_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    switch (p->x_dtype) {
    case CANON_DTYPE_F32: launch_update_parts<CANON_DTYPE_F32>(pp, s); break;
    case CANON_DTYPE_BF16: launch_update_parts<CANON_DTYPE_BF16>(pp, s); break;
    default: launch_update_parts<CANON_DTYPE_F16>(pp, s); break;
    }
    return check_launch("canon_conv1d_update_parts");
}

const char *canon_conv1d_fwd_parts_plan(const canon_conv1d_fwd_params *p, const canon_conv1d_part *parts, int32_t nparts)
{
    FwdPartsPlan pp;
    if (plan_fwd_parts(p, parts, nparts, &pp) != CANON_OK) return nullptr;
    return pp.single ? "blc_vec_parts" : "per_part";
}

const char *canon_conv1d_update_parts_plan(const canon_conv1d_update_params *p, const canon_conv1d_part *parts,
                                           int32_t nparts)
{
    UpdPartsPlan pp;
    if (plan_update_parts(p, parts, nparts, &pp) != CANON_OK) return nullptr;
    return pp.single ? "update_vec_parts" : "per_part";
}

}  // extern "C"
