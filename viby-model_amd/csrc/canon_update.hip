// Canon causal depthwise conv1d for MI355X (gfx950): the single-token decode
// update kernels (in-place shift-register conv_state) and their launchers.
#include "canon_device.h"

namespace canon {

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

template <int DT, int W, int S, int NB, bool POOL = false>
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
    uint32_t srow[NB];   // conv_state row of each batch entry
#pragma unroll
    for (int n = 0; n < NB; ++n) {
        const uint32_t b = bg * NB + n;
        tm[n] = 1.0f;
        if (b < a.B) {
            X[n] = *(const uint4 *)(a.x + ((int64_t)b * a.x_sb + c0) * BY);
            srow[n] = POOL ? (uint32_t)a.indices[b] : b;   // POOL: rows of a state pool (conv_state_indices)
            const uint4 *sp = (const uint4 *)(a.state + ((int64_t)srow[n] * a.s_sb + (int64_t)c0 * S) * BY);
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
        uint4 *dp = (uint4 *)(a.state + ((int64_t)srow[n] * a.s_sb + (int64_t)c0 * S) * BY);
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

// the same with batch entry b using row conv_state_indices[b] of a state pool
template <int DT, int W, int S, int NB>
__global__ __launch_bounds__(256) void canon_update_vec_pool_kernel(const UpdArgs a)
{
    update_vec_block<DT, W, S, NB, true>(a, blockIdx.x);
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
    const uint32_t srow = a.indices ? (uint32_t)a.indices[b] : b;
    const int64_t so = (int64_t)srow * a.s_sb + (int64_t)c * a.s_sc;
    // circular-buffer mode: the token goes to slot pos, the W-1 slots before it (cyclically) are the history
    int pos = -1;
    if (a.seqlens) {
        pos = a.seqlens[b] % S;
        if (pos < 0) pos += S;
    }
    const float xr = load1<DT>(a.x, (int64_t)b * a.x_sb + (int64_t)c * a.x_sc);
    float xt = xr;
    if (a.tmask) xt = mul_round<DT>(xr, load_mask(a.tmask, (int64_t)b * a.m_sb, a.mask_dtype));
    for (int k = 0; k < W - 1; ++k) {
        int slot = S - (W - 1) + k;
        if (pos >= 0) {
            slot = pos - (W - 1) + k;
            if (slot < 0) slot += S;
        }
        win[4 - W + k] = load1<DT>(a.state, so + (int64_t)slot * a.s_ss);
    }
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
    if (pos >= 0) {
        store1<DT>(a.state, so + (int64_t)pos * a.s_ss, xt);
        return;
    }
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
// launch
// ---------------------------------------------------------------------------
namespace {

template <int DT, int W, int NB> void launch_update_vec_nb(const UpdPlan &pl, hipStream_t s)
{
    const dim3 g(pl.grid), b(256);
    if (pl.args.indices) {
        switch (pl.args.S) {
        case 3: hipLaunchKernelGGL((canon_update_vec_pool_kernel<DT, W, 3, NB>), g, b, 0, s, pl.args); break;
        case 4: hipLaunchKernelGGL((canon_update_vec_pool_kernel<DT, W, 4, NB>), g, b, 0, s, pl.args); break;
        default: hipLaunchKernelGGL((canon_update_vec_pool_kernel<DT, W, 8, NB>), g, b, 0, s, pl.args); break;
        }
        return;
    }
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

template <int DT, int NB> void launch_update_parts_nb(const PartTable<UpdArgs> &m, int S, uint32_t grid, hipStream_t s)
{
    const dim3 g(grid), b(256);
    switch (S) {
    case 3: hipLaunchKernelGGL((canon_update_vec_parts_kernel<DT, 4, 3, NB>), g, b, 0, s, m); break;
    case 4: hipLaunchKernelGGL((canon_update_vec_parts_kernel<DT, 4, 4, NB>), g, b, 0, s, m); break;
    default: hipLaunchKernelGGL((canon_update_vec_parts_kernel<DT, 4, 8, NB>), g, b, 0, s, m); break;
    }
}

template <int DT> void launch_update_parts_t(const UpdPartsPlan &pp, hipStream_t s)
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

}  // namespace

void launch_update(const UpdPlan &pl, int x_dtype, hipStream_t s)
{
    switch (x_dtype) {
    case CANON_DTYPE_F32: launch_update<CANON_DTYPE_F32>(pl, s); break;
    case CANON_DTYPE_BF16: launch_update<CANON_DTYPE_BF16>(pl, s); break;
    default: launch_update<CANON_DTYPE_F16>(pl, s); break;
    }
}

void launch_update_parts(const UpdPartsPlan &pp, int x_dtype, hipStream_t s)
{
    switch (x_dtype) {
    case CANON_DTYPE_F32: launch_update_parts_t<CANON_DTYPE_F32>(pp, s); break;
    case CANON_DTYPE_BF16: launch_update_parts_t<CANON_DTYPE_BF16>(pp, s); break;
    default: launch_update_parts_t<CANON_DTYPE_F16>(pp, s); break;
    }
}

}  // namespace canon
