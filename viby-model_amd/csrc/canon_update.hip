// Canon causal depthwise conv1d for MI355X (gfx950): the single-token decode
// update kernels (in-place shift-register conv_state) and their launchers.
#include "canon_device.h"

namespace canon {

// Row of the state pool that batch entry b uses (conv_state_indices), or kSkipRow when the index lies outside
// the pool (negative, or not below state_rows when the caller stated the pool's size): such an entry is
// left alone -- no state row and no output is touched.
constexpr uint32_t kSkipRow = 0xFFFFFFFFu;
__device__ __forceinline__ uint32_t pool_row(const UpdArgs &a, uint32_t b)
{
    const int32_t i = a.indices[b];
    if (i < 0 || (a.state_rows > 0 && (uint32_t)i >= a.state_rows)) return kSkipRow;
    return (uint32_t)i;
}

// ---------------------------------------------------------------------------
// decode update, vectorised: contiguous [B, C, S] state, channel-contiguous
// x / out.  One lane owns the state rows of E adjacent channels, E chosen so
// that they are ONE run of at most 16 bytes (16-bit: two channels for S = 3 or
// 4, one for S = 8; fp32: one channel, 32 bytes for S = 8): a wave then reads
// and writes one dense stretch of the state per instruction, which is what
// the memory pipeline wants -- wider lanes (eight channels each, the lanes of
// a wave 48..128 bytes apart) ran 1.5-2x slower.  The lane computes its E
// outputs and writes the run back shifted by one element per channel with the
// new token in the last slot: one fused gather / shift / write, no second
// pass.  Each lane walks NB batch rows so the taps are fetched once per NB
// tokens.
// ---------------------------------------------------------------------------
// One output of the eager module's step (rounding mode "eager"): history taken from packed state words
// starting at element `first`, the token last.
template <int DT, int W>
__device__ __forceinline__ float eager_step(const float *w, float bias, const uint32_t *state_words, int first, float xt, bool act)
{
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < W - 1; ++k)
        s = __fadd_rn(s, mul_round<DT>(Packed<DT>::as_float(Packed<DT>::get(state_words, first + k)), w[k]));
    s = __fadd_rn(s, mul_round<DT>(xt, w[W - 1]));
    s = round_result<DT>(s);
    float acc = round_result<DT>(__fadd_rn(bias, s));
    if (act) acc = round_result<DT>(silu_precise(acc));
    return acc;
}

template <int DT, int W, int S, int NB, int MODE, bool POOL>
__device__ __forceinline__ void update_vec_body(const UpdArgs &a, const uint32_t bg, const uint32_t c0,
                                                const uint32_t (*X)[(upd_lane_channels(Elem<DT>::bytes, S) * Elem<DT>::bytes + 3) / 4],
                                                const uint32_t (*ST)[upd_lane_channels(Elem<DT>::bytes, S) * S * Elem<DT>::bytes / 4],
                                                const uint32_t *srow)
{
    constexpr int BY = Elem<DT>::bytes;
    constexpr int E = upd_lane_channels(BY, S);
    constexpr int ND = E * S * BY / 4;
    constexpr int NX = (E * BY + 3) / 4;
    constexpr int WDT = MODE == TAPS_WIDE ? CANON_DTYPE_F32 : DT;      // weight type of the straight-line modes

    TapWords<WDT, E> tw;
    RawTaps<E> raw;
    if constexpr (MODE == TAPS_ANY) {
        fetch_taps<W, E>(a.weight, a.bias, a.w_sc, a.w_sk, a.w_dtype, a.w_vec != 0, c0, raw);
    } else {
        static_assert(MODE == TAPS_ANY || W == 4, "the contiguous tap layouts are [C, 4]");
        fetch_taps_contiguous<WDT, E>(a.weight, a.bias, c0, tw);
    }
    float tm[NB];
#pragma unroll
    for (int n = 0; n < NB; ++n) tm[n] = 1.0f;
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
    if constexpr (MODE == TAPS_ANY) decode_taps<DT, W, E>(raw, a.w_dtype, a.w_vec != 0, a.bias != nullptr, w, bias);
    else decode_taps_contiguous<DT, WDT, E>(tw, a.bias != nullptr, w, bias);

#pragma unroll
    for (int n = 0; n < NB; ++n) {
        const uint32_t b = bg * NB + n;
        if (b >= a.B || (POOL && srow[n] == kSkipRow)) continue;
        float xr[E], xt[E], o[E];
#pragma unroll
        for (int e = 0; e < E; ++e) xr[e] = Packed<DT>::as_float(Packed<DT>::get(X[n], e));
        if (a.tmask) {
#pragma unroll
            for (int e = 0; e < E; ++e) xt[e] = mul_round<DT>(xr[e], tm[n]);
        } else {
#pragma unroll
            for (int e = 0; e < E; ++e) xt[e] = xr[e];
        }
        if (!a.eager) {
#pragma unroll
            for (int e = 0; e < E; ++e) {
                float acc = bias[e];
#pragma unroll
                for (int k = 0; k < W - 1; ++k)
                    acc = fmaf(w[e][k], Packed<DT>::as_float(Packed<DT>::get(ST[n], e * S + (S - (W - 1) + k))), acc);
                o[e] = fmaf(w[e][W - 1], xt[e], acc);
            }
            if (a.act) {
#pragma unroll
                for (int e = 0; e < E; ++e) o[e] = silu_fast(o[e]);
            }
        } else {
            // the eager module's step: every product rounded to the storage type, their fp32 sum rounded, then
            // the bias added and rounded, then the activation rounded
#pragma unroll
            for (int e = 0; e < E; ++e) o[e] = eager_step<DT, W>(w[e], bias[e], &ST[n][0], e * S + (S - (W - 1)), xt[e], a.act != 0);
        }
        if (a.res_mode == CANON_RESIDUAL_MASKED) {
#pragma unroll
            for (int e = 0; e < E; ++e) o[e] = __fadd_rn(o[e], xt[e]);
        } else if (a.res_mode == CANON_RESIDUAL_UNMASKED) {
#pragma unroll
            for (int e = 0; e < E; ++e) o[e] = __fadd_rn(o[e], xr[e]);
        }
        uint32_t ow[NX] = {};
#pragma unroll
        for (int e = 0; e < E; ++e) Packed<DT>::put(ow, e, Packed<DT>::raw_of(o[e]));
        char *op = a.out + ((int64_t)b * a.o_sb + c0) * BY;
        if constexpr (E * BY == 2) *(uint16_t *)op = (uint16_t)ow[0];
        else store_words<NX>(op, ow);

        // new run: element (e, k) <- old (e, k+1); (e, S-1) <- token (its own bits unless a mask scaled it)
        uint32_t nw[ND] = {};
#pragma unroll
        for (int e = 0; e < E; ++e) {
#pragma unroll
            for (int k = 0; k < S - 1; ++k) Packed<DT>::put(nw, e * S + k, Packed<DT>::get(ST[n], e * S + k + 1));
            const uint32_t tok = a.tmask ? Packed<DT>::raw_of(xt[e]) : Packed<DT>::get(X[n], e);
            Packed<DT>::put(nw, e * S + S - 1, tok);
        }
        store_words<ND>(a.state + ((int64_t)srow[n] * a.s_sb + (int64_t)c0 * S) * BY, nw);
    }
}

// What a lane needs to request its token and its state rows.  The plain kernel gets these as leading scalar
// arguments, which arrive in registers with the wave (kernel-argument preload), requests the data from them and
// reads its argument block while those loads are on their way; the pool and multi-part kernels read the block
// first and fill this from it.
struct UpdLead {
    const char *x;
    char *state;
    int64_t x_sb, s_sb;
    uint32_t nthreads, nvec, B;
    FastDiv div_nvec;
};

__device__ __forceinline__ UpdLead lead_of(const UpdArgs &a)
{
    return UpdLead{a.x, a.state, a.x_sb, a.s_sb, a.nthreads, a.nvec, a.B, a.div_nvec};
}

template <int DT, int W, int S, int NB, bool POOL = false, typename ARGS>
__device__ __forceinline__ void update_vec_block(const ARGS &args, const UpdLead &h, const uint32_t blk)
{
    constexpr int BY = Elem<DT>::bytes;
    constexpr int E = upd_lane_channels(BY, S);
    constexpr int ND = E * S * BY / 4;          // words of state per lane and batch entry
    constexpr int NX = (E * BY + 3) / 4;        // words of token / output
    static_assert(E * S * BY % 4 == 0, "a lane's piece of the state must be whole words");
    static_assert(!(POOL && ARGS::kLate), "the pool indices are part of the argument block");
    const uint32_t tid = blk * 256u + threadIdx.x;
    if (tid >= h.nthreads) return;
    const uint32_t bg = fdiv(tid, h.div_nvec);
    const uint32_t cv = tid - bg * h.nvec;
    const uint32_t c0 = cv * E;

    uint32_t X[NB][NX];
    uint32_t ST[NB][ND];
    uint32_t srow[NB];   // conv_state row of each batch entry
    if constexpr (ARGS::kLate) {
#pragma unroll
        for (int n = 0; n < NB; ++n) {
            const uint32_t b = bg * NB + n;
            srow[n] = b;
            if (b < h.B) {
                const char *xp = h.x + ((int64_t)b * h.x_sb + c0) * BY;
                if constexpr (E * BY == 2) X[n][0] = *(const uint16_t *)xp;
                else load_words<NX>(xp, X[n]);
                load_words<ND>(h.state + ((int64_t)b * h.s_sb + (int64_t)c0 * S) * BY, ST[n]);
            }
        }
    }
    const UpdArgs &a = args.get();
    if constexpr (!ARGS::kLate) {
        // the test reads a field of each 64-byte line of the arguments this kernel uses (the divisor is never 0,
        // the flag never negative), so that all are requested together instead of one after the other
        if ((a.div_nvec.d == 0) | (a.w_vec < 0)) return;   // '|': one test, no short circuit
#pragma unroll
        for (int n = 0; n < NB; ++n) {
            const uint32_t b = bg * NB + n;
            srow[n] = b;
            if (b < a.B) {
                // POOL: rows of a state pool (conv_state_indices); an entry whose index is outside the pool is
                // skipped (nothing of it is read or written)
                if constexpr (POOL) {
                    srow[n] = pool_row(a, b);
                    if (srow[n] == kSkipRow) continue;
                }
                const char *xp = a.x + ((int64_t)b * a.x_sb + c0) * BY;
                if constexpr (E * BY == 2) X[n][0] = *(const uint16_t *)xp;
                else load_words<NX>(xp, X[n]);
                load_words<ND>(a.state + ((int64_t)srow[n] * a.s_sb + (int64_t)c0 * S) * BY, ST[n]);
            }
        }
    }
    if constexpr (W == 4) {
        if (a.tap_mode == TAPS_SAME) {
            update_vec_body<DT, W, S, NB, TAPS_SAME, POOL>(a, bg, c0, X, ST, srow);
            return;
        }
        if constexpr (DT != CANON_DTYPE_F32) {
            if (a.tap_mode == TAPS_WIDE) {
                update_vec_body<DT, W, S, NB, TAPS_WIDE, POOL>(a, bg, c0, X, ST, srow);
                return;
            }
        }
    }
    update_vec_body<DT, W, S, NB, TAPS_ANY, POOL>(a, bg, c0, X, ST, srow);
}

// The leading scalars (fourteen dwords: they arrive in registers) listed once, for the kernel's signature and for the
// struct that mirrors the kernel-argument segment, through which the argument block behind them is read late.
#define CANON_UPD_LEAD(X)                                                                                         \
    X(const char *, x) X(char *, state) X(int64_t, x_sb) X(int64_t, s_sb) X(uint32_t, nthreads) X(uint32_t, nvec) \
    X(uint32_t, B) X(uint32_t, div_m) X(uint32_t, div_s1) X(uint32_t, div_s2)
struct UpdSegment {
    CANON_UPD_LEAD(CANON_LEAD_FIELD)
    UpdArgs a;
};
static_assert(offsetof(UpdSegment, a) == 14 * 4, "fourteen leading dwords, then the argument block");

template <int DT, int W, int S, int NB>
__global__ __launch_bounds__(256) void canon_update_vec_kernel(CANON_UPD_LEAD(CANON_LEAD_PARAM) const UpdArgs a)
{
    const UpdLead h = {x, state, x_sb, s_sb, nthreads, nvec, B, FastDiv{nvec, div_m, div_s1, div_s2}};
#ifdef CANON_NO_LATE_ARGS
    update_vec_block<DT, W, S, NB>(ArgsRead<UpdArgs>{a}, h, blockIdx.x);
#else
    update_vec_block<DT, W, S, NB>(ArgsToRead<UpdArgs>{(uint32_t)offsetof(UpdSegment, a)}, h, blockIdx.x);
#endif
}

// the same with batch entry b using row conv_state_indices[b] of a state pool
template <int DT, int W, int S, int NB>
__global__ __launch_bounds__(256) void canon_update_vec_pool_kernel(const UpdArgs a)
{
    update_vec_block<DT, W, S, NB, true>(ArgsRead<UpdArgs>{a}, lead_of(a), blockIdx.x);
}

// the token of one step given as several channel ranges (separate projections), one launch
template <int DT, int W, int S, int NB>
__global__ __launch_bounds__(256) void canon_update_vec_parts_kernel(uint32_t fb1, uint32_t fb2, uint32_t fb3,
                                                                     const PartTable<UpdArgs> m)
{
    // fb1..fb3: the first blocks of parts 1..3 once more as leading scalars, which arrive in registers with the
    // wave (the block knows its part without a first read of the table); the part's arguments are copied, so
    // that their loads are issued together.
    const uint32_t blk = blockIdx.x;
    const uint32_t p = (blk >= fb1 ? 1u : 0u) + (blk >= fb2 ? 1u : 0u) + (blk >= fb3 ? 1u : 0u);
    const uint32_t first = p == 0 ? 0u : (p == 1 ? fb1 : (p == 2 ? fb2 : fb3));
    const UpdArgs a = m.part[p];
    update_vec_block<DT, W, S, NB>(ArgsRead<UpdArgs>{a}, lead_of(a), blk - first);
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
    const uint32_t srow = a.indices ? pool_row(a, b) : b;
    if (srow == kSkipRow) return;
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
        acc = finish<DT>(acc, a.act, a.res_mode, 0, xt, xr);
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
    const UpdArgs &a = pl.args;
#define CANON_UPD_LAUNCH(SS)                                                                                            \
    hipLaunchKernelGGL((canon_update_vec_kernel<DT, W, SS, NB>), g, b, 0, s, a.x, a.state, a.x_sb, a.s_sb, a.nthreads,   \
                       a.nvec, a.B, a.div_nvec.m, a.div_nvec.s1, a.div_nvec.s2, a)
    switch (a.S) {
    case 3: CANON_UPD_LAUNCH(3); break;
    case 4: CANON_UPD_LAUNCH(4); break;
    default: CANON_UPD_LAUNCH(8); break;
    }
#undef CANON_UPD_LAUNCH
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
    case 3: hipLaunchKernelGGL((canon_update_vec_parts_kernel<DT, 4, 3, NB>), g, b, 0, s, m.first_block[1], m.first_block[2], m.first_block[3], m); break;
    case 4: hipLaunchKernelGGL((canon_update_vec_parts_kernel<DT, 4, 4, NB>), g, b, 0, s, m.first_block[1], m.first_block[2], m.first_block[3], m); break;
    default: hipLaunchKernelGGL((canon_update_vec_parts_kernel<DT, 4, 8, NB>), g, b, 0, s, m.first_block[1], m.first_block[2], m.first_block[3], m); break;
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

// Asking for a kernel's attributes makes the runtime load this file's code object onto the current device.
hipError_t preload_update()
{
    hipFuncAttributes attr;
    return hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(&(canon_update_generic_kernel<CANON_DTYPE_F32>)));
}

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
