// Canon causal depthwise conv1d for MI355X (gfx950, wave64): the prefill kernels
// (time-contiguous, channel-contiguous, strided) and their launchers.
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
#include "canon_device.h"

namespace canon {

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
// One element of the row computed on its own (the few elements of a row that do not fill an aligned
// 16-byte vector, see EDGE below): scalar loads of its window, same arithmetic.  The loads are
// issued with the row's vector loads (bcl_edge_issue) and consumed after the vector work
// (bcl_edge_finish), so they cost the wave no round trip of their own.
struct EdgeWindow {
    float x[4];   // raw x[t-3 .. t] (0 where t-3+k < 0 and there is no initial state)
    float m[4];   // their mask entries
};

template <int DT, int W, bool MASK>
__device__ __forceinline__ void bcl_edge_issue(const FwdArgs &a, const char *xrow, uint32_t b, uint32_t c, int64_t t,
                                               EdgeWindow &e)
{
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        e.x[k] = 0.0f;
        e.m[k] = 1.0f;
    }
#pragma unroll
    for (int k = 4 - W; k < 4; ++k) {
        const int64_t tt = t - 3 + k;
        if (tt >= 0) e.x[k] = load1<DT>(xrow, tt);
        else if (a.init) e.x[k] = load1<DT>(a.init, b * a.i_sb + c * a.i_sc + (a.S_in + tt) * a.i_ss);
    }
    if constexpr (MASK) {
        // the four entries as one run from max(t-3, 0) (rows are at least 16 vectors long)
        const int64_t first = t - 3 > 0 ? t - 3 : 0;
        const int shift = (int)(first - (t - 3));   // 0 .. 3 window slots lie before the row
        int64_t base[1] = {b * a.m_sb + first * a.m_sl};
        float run[1][4];
        load_mask_vec<4, 1>(a.mask, base, a.m_sl, a.mask_dtype, false, run);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int j = k - shift;
            e.m[k] = j == 0 ? run[0][0] : j == 1 ? run[0][1] : j == 2 ? run[0][2] : j == 3 ? run[0][3] : 1.0f;
        }
    }
}

template <int DT, int W, bool MASK>
__device__ __forceinline__ void bcl_edge_finish(const FwdArgs &a, const float (*w)[W], float bv, char *orow, int64_t t,
                                                const EdgeWindow &e)
{
    float win[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        win[k] = e.x[k];
        if constexpr (MASK) {
            if (t - 3 + k >= 0) win[k] = mul_round<DT>(e.x[k], e.m[k]);   // history from the initial state is not masked
        }
    }
    float acc = bv;
#pragma unroll
    for (int k = 0; k < W; ++k) acc = fmaf(w[0][k], win[(4 - W) + k], acc);
    store1<DT>(orow, t, finish<DT>(acc, a.act, a.res_mode, a.eager, win[3], e.x[3]));
}

// Activation, residual and store of one 16-byte vector of accumulators.
template <int DT, bool MASK, bool EAGER>
__device__ __forceinline__ void bcl_finish_vec(const FwdArgs &a, float *o, const float *xr, const float *xm, char *dst, bool write)
{
    constexpr int E = Elem<DT>::per_vec;
    activate<DT, E>(o, a.act != 0, EAGER);
    if (a.res_mode == CANON_RESIDUAL_UNMASKED || (!MASK && a.res_mode)) {
#pragma unroll
        for (int j = 0; j < E; ++j) o[j] += xr[j];
    } else if (a.res_mode == CANON_RESIDUAL_MASKED) {
#pragma unroll
        for (int j = 0; j < E; ++j) o[j] += xm[j];
    }
    if (write) store_vec<true>(dst, pack_vec<DT>(o));
}

// EDGE: the rows are contiguous in time but do not start on 16-byte boundaries (a length or a
// row stride that is not a multiple of E).  The aligned middle of every row runs through the
// same vector code, shifted by `head` elements; the up to E-1 elements before it and after it
// are computed one per lane by the waves that own the first and the last segment.
//
// The scalars in front of the argument block are what a wave needs to request its row.  Scalar kernel
// arguments at the head of the list arrive in registers with the wave (kernel-argument preload: the library is
// built with -mllvm -amdgpu-kernarg-preload-count), an aggregate does not, so the row loads are issued without
// waiting for a read of the argument block; everything else is read from the block while they are in flight.
// Measured at B 8, C 3456, L 1024, bf16: 20.3 -> 19.6 us, half of it from the preload and half from the
// scalars sharing one line of the argument segment.  (The channel-contiguous prefill and the decode update
// gained nothing from the same change, or lost: they take their arguments as one block.)
// `wpb`: waves per block, 1, 4 or 8 (the waves are independent; large unmasked launches run 0.5-1 % faster in
// blocks of 8: 19.6 -> 19.5 us at B 8, 70.0 -> 69.1 us at B 32; 16 are 7 % slower; with a mask 8 are 6-9 % slower
// and single waves 1-2 % faster than blocks of 4).
template <int DT, int W, int U, bool MASK, bool BIG, bool EDGE = false>
__global__ __launch_bounds__(64 * kBclMaxWaves) void canon_fwd_bcl_kernel(const char *x_base, int64_t x_sb, int64_t x_sc,
                                                                          uint32_t ntasks, uint32_t nseg, uint32_t C,
                                                                          uint32_t divC_m, uint32_t divC_s1, uint32_t divC_s2,
                                                                          uint32_t nvec_row, uint32_t wpb, const FwdArgs a)
{
    constexpr int E = Elem<DT>::per_vec;
    const int lane = threadIdx.x & 63;
    const uint32_t task = __builtin_amdgcn_readfirstlane(blockIdx.x * wpb + (threadIdx.x >> 6));
    if (task >= ntasks) return;
    uint32_t row = task, seg = 0;
    if (nseg == 2) {          // (from the leading scalars alone: no read of the argument block before the row loads)
        row = task >> 1;
        seg = task & 1u;
    } else if (nseg > 1) {
        row = fdiv(task, a.div_nseg);
        seg = task - row * nseg;
    }
    const FastDiv div_C = {C, divC_m, divC_s1, divC_s2};
    const uint32_t b = fdiv(row, div_C);
    const uint32_t c = row - b * C;

    const int64_t row_off = (int64_t)b * x_sb + (int64_t)c * x_sc;   // in elements; the same for x and out
    const char *xrow = x_base + row_off * Elem<DT>::bytes;
    char *orow = a.out + ((int64_t)b * a.o_sb + (int64_t)c * a.o_sc) * Elem<DT>::bytes;
    const uint32_t v0 = seg * (64u * U) + lane;
    // head: elements of the row before its first aligned vector; nvec: aligned vectors of this row
    uint32_t head = 0, nvec = nvec_row;
    if constexpr (EDGE) {
        head = (uint32_t)((E - (row_off % E)) % E);
        if (head > a.L) head = a.L;
        nvec = (a.L - head) / E;
    }
    const char *xvec = xrow + (int64_t)head * Elem<DT>::bytes;   // 16-byte aligned
    char *ovec = orow + (int64_t)head * Elem<DT>::bytes;

    // row data first (the long latency), then the taps (scalar-cache hits)
    uint4 X[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t v = v0 + u * 64u;
        X[u] = make_uint4(0, 0, 0, 0);
        if (v < nvec) X[u] = load_vec<true>(xvec + (int64_t)v * 16);
    }
    // a later segment's history: the vector before the segment, requested by lane 0 together with the segment itself
    // (the wave of the segment before requests the same vector at about the same time)
    uint4 P = make_uint4(0, 0, 0, 0);
    constexpr bool kPrevVector = !MASK && !EDGE;
    if constexpr (kPrevVector) {
        if (seg > 0 && lane == 0) P = load_vec<false>(xvec + ((int64_t)v0 - 1) * 16);
    }

    // EDGE: lanes 0 .. head-1 of the first segment take the elements before the first vector,
    // lanes 32 .. 32+tail-1 of the last segment the elements after the last one
    EdgeWindow edge;
    int64_t edge_t = -1;
    if constexpr (EDGE) {
        const uint32_t tail = a.L - head - nvec * E;
        if (seg == 0 && (uint32_t)lane < head) edge_t = lane;
        if (seg == a.nseg - 1 && lane >= 32 && (uint32_t)(lane - 32) < tail) edge_t = (int64_t)head + (int64_t)nvec * E + (lane - 32);
        if (edge_t >= 0) bcl_edge_issue<DT, W, MASK>(a, xrow, b, c, edge_t, edge);
    }

    RawTaps<1> raw;
    fetch_taps_uniform<W>(a.weight, a.bias, a.w_sc, a.w_sk, a.w_dtype, a.w_vec != 0, a.b_pair != 0, c, raw);

    // all mask entries of the segment, requested before anything is consumed; the masked inputs are formed
    // at once and kept in storage format (XM): eight mask floats per vector held until the main loop would
    // cost the kernel a wave per SIMD
    uint4 XM[MASK ? U : 1];
    if constexpr (MASK) {
        float M[U][E];
        int64_t mbase[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t v = v0 + u * 64u;
            // idle lanes shadow the last vector (a row without any aligned vector reads from its start)
            const int64_t vv = v < nvec ? v : (nvec ? nvec - 1u : 0u);
            mbase[u] = b * a.m_sb + ((int64_t)head + vv * E) * a.m_sl;
            if constexpr (EDGE) {
                if (nvec == 0) mbase[u] = b * a.m_sb;
            }
        }
        load_mask_vec<E, U>(a.mask, mbase, a.m_sl, a.mask_dtype, !EDGE && a.m_vec != 0, M);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float xr[E], xm[E];
            unpack_vec<DT>(X[u], xr);
#pragma unroll
            for (int j = 0; j < E; ++j) xm[j] = mul_round<DT>(xr[j], M[u][j]);
            XM[u] = pack_vec<DT>(xm);   // exact: the products are already rounded to the storage type
        }
    }

    float w[1][W], bvv[1];
    decode_taps<DT, W, 1>(raw, a.w_dtype, a.w_vec != 0, a.bias != nullptr, w, bvv);
    const float bv = bvv[0];

    // history of the segment's first vector (only lane 0's copy is consumed)
    float carry[3] = {0.0f, 0.0f, 0.0f};
    if (kPrevVector && seg > 0) {
        float pv[E];
        unpack_vec<DT>(P, pv);
#pragma unroll
        for (int j = 0; j < 3; ++j)
            if (j >= 3 - (W - 1)) carry[j] = pv[E - 3 + j];
    } else if (lane == 0) {
        if (seg > 0 || (EDGE && head > 0)) {
            const int64_t t0 = (int64_t)head + (int64_t)v0 * E;
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                const int64_t t = t0 - 3 + j;
                if (j < 3 - (W - 1)) continue;
                if (t >= 0) {
                    float v = load1<DT>(xrow, t);
                    if constexpr (MASK) v = mul_round<DT>(v, load_mask(a.mask, b * a.m_sb + t * a.m_sl, a.mask_dtype));
                    carry[j] = v;
                } else if (a.init) {
                    carry[j] = load1<DT>(a.init, b * a.i_sb + c * a.i_sc + (a.S_in + t) * a.i_ss);
                }
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
        if constexpr (MASK) unpack_vec<DT>(XM[u], xm);
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
        // the rounding mode is branched on around the whole epilogue, store included, so that the eager module's
        // extra roundings are not evaluated and then discarded (selects) on the usual path
        if (a.eager) bcl_finish_vec<DT, MASK, true>(a, o, xr, xm, ovec + (int64_t)v * 16, v < nvec);
        else bcl_finish_vec<DT, MASK, false>(a, o, xr, xm, ovec + (int64_t)v * 16, v < nvec);
    }

    if constexpr (EDGE) {
        if (edge_t >= 0) bcl_edge_finish<DT, W, MASK>(a, w, bv, orow, edge_t, edge);
    }

    if (a.fin && seg == a.nseg - 1) capture_row_state<DT>(a, b, c, lane);
}

// ---------------------------------------------------------------------------
// prefill, time-contiguous rows of at most 32 vectors (whole vectors, 16-byte
// aligned): a row takes P = 1, 2, 4, .. 32 adjacent lanes of a wave (the next
// power of two from its vector count) and a wave 64 / P rows, so short prompts
// keep most lanes busy and every access is a 16-byte one.  A lane's history is
// its left neighbour's last three inputs (wave shift) unless it holds the
// first vector of its row; the rows of a wave belong to different channels, so
// each lane loads its own taps.  Field use: nseg = P, chunk = log2(P),
// ntasks = rows (B * C), nvec = vectors per row.
// ---------------------------------------------------------------------------
template <int DT, int W, bool MASK>
__global__ __launch_bounds__(256) void canon_fwd_bcl_short_kernel(const FwdArgs a)
{
    constexpr int E = Elem<DT>::per_vec;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * 4u + (threadIdx.x >> 6));
    const uint32_t shift = a.chunk, P = a.nseg;
    const uint32_t first_row = wave * (64u >> shift);
    if (first_row >= a.ntasks) return;
    const uint32_t sub = lane & (P - 1u);
    const uint32_t row = first_row + (lane >> shift);
    const bool row_ok = row < a.ntasks;
    const uint32_t rr = row_ok ? row : a.ntasks - 1u;            // idle lanes shadow the last row / vector:
    const uint32_t v = sub < a.nvec ? sub : a.nvec - 1u;         // loads need no predicate
    const bool active = row_ok && sub < a.nvec;
    const uint32_t b = fdiv(rr, a.div_C);
    const uint32_t c = rr - b * a.C;
    const char *xrow = a.x + ((int64_t)b * a.x_sb + (int64_t)c * a.x_sc) * Elem<DT>::bytes;
    char *orow = a.out + ((int64_t)b * a.o_sb + (int64_t)c * a.o_sc) * Elem<DT>::bytes;

    const uint4 X = load_vec<true>(xrow + (int64_t)v * 16);
    RawTaps<1> raw;
    fetch_taps<W, 1>(a.weight, a.bias, a.w_sc, a.w_sk, a.w_dtype, a.w_vec != 0, c, raw);
    float M[1][E];
    if constexpr (MASK) {
        const int64_t mbase[1] = {(int64_t)b * a.m_sb + (int64_t)v * E * a.m_sl};
        load_mask_vec<E, 1>(a.mask, mbase, a.m_sl, a.mask_dtype, a.m_vec != 0, M);
    }
    float w[1][W], bvv[1];
    decode_taps<DT, W, 1>(raw, a.w_dtype, a.w_vec != 0, a.bias != nullptr, w, bvv);
    const float bv = bvv[0];

    float xr[E], xm_store[MASK ? E : 1];
    float *xm = MASK ? xm_store : xr;
    unpack_vec<DT>(X, xr);
    if constexpr (MASK) {
#pragma unroll
        for (int j = 0; j < E; ++j) xm[j] = mul_round<DT>(xr[j], M[0][j]);
    }
    // seq[0..2] = the three masked inputs before this vector
    float seq[E + 3];
    seq[0] = wave_shift_up(xm[E - 3], 0.0f);
    seq[1] = wave_shift_up(xm[E - 2], 0.0f);
    seq[2] = wave_shift_up(xm[E - 1], 0.0f);
    if (sub == 0) {
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            seq[j] = 0.0f;
            if (j >= 3 - (W - 1) && a.init)
                seq[j] = load1<DT>(a.init, b * a.i_sb + c * a.i_sc + (int64_t)(a.S_in - 3 + j) * a.i_ss);
        }
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
    if (a.eager) bcl_finish_vec<DT, MASK, true>(a, o, xr, xm, orow + (int64_t)v * 16, active);
    else bcl_finish_vec<DT, MASK, false>(a, o, xr, xm, orow + (int64_t)v * 16, active);

    if (a.fin && row_ok)
        for (uint32_t slot = sub; slot < (uint32_t)a.S_out; slot += P) capture_row_state<DT>(a, b, c, (int)slot);
}

// ---------------------------------------------------------------------------
// prefill, channel-contiguous rows ([B, L, C] memory, x_stride_c == 1): the
// layout CanonLayer hands over (a transposed view of [B, T, D]).
//
// One lane owns E adjacent channels (VB = 8 bytes of every row: 4 x 16-bit or
// 2 x fp32; 16-byte lanes need 142 registers and measured 4-9 % slower) and R
// consecutive time steps; the WT waves of a block own WT consecutive R-row
// slabs of the same 64-lane channel tile, so a block streams a
// [WT * R rows] x [512 B] tile (short-lived waves over a compact window:
// measured to be what HBM wants; long per-lane time runs lose 10-20 %).
// Memory is reached through buffer resources, one per tensor and wave: the
// row is a scalar offset and the lane a 32-bit vector offset, so an access
// costs no 64-bit address arithmetic, and lanes past the last channel are
// dropped by the range check of the resource.
// The three rows a wave needs from before its slab are the last three rows of
// the previous wave: each wave publishes the raw tail of its slab in LDS, one
// barrier, the next wave picks it up -- only the first wave of a block reads
// its history from memory, and the block order makes that a hit in the L2 of
// its XCD (see blc_block_linear).  The same barrier passes on the taps: the
// waves of a tile fetch a WT-th of its taps and bias each (every wave fetching
// all of them cost 3 % at B = 32: 2.5 KB of L2 traffic per 8 KB of x).
// All loads (history, slab, taps) are issued before the first wait on data.
// The plain kernel requests history and slab before it has read its argument
// block (from leading scalar arguments that arrive in registers), which takes
// the read of the block out of the way: 3 % with a mask, 5-22 % at C 640 /
// 960.  In large launches it requests the taps even before those, through
// two pointers it reads ahead of the block (see blc_block_body).
// ---------------------------------------------------------------------------
// One row of a slab: out = act(bias + taps . (history, x)) (+ residual), written through the wave's buffer
// resource.  ACT / RES / EAGER: the activation flag, the residual mode and the rounding mode when they are
// known at compile time (-1: read from the arguments; a select per element and a branch per row then).
// keep0..2 (wave uniform): whether the rows t-3, t-2, t-1 belong to the packed sequence of row t
// (always true without seq_idx); a row of another sequence enters as zeros.
template <int DT, int W, bool MASK, bool BIG, int VB, int ACT = -1, int RES = -1, int EAGER = -1>
__device__ __forceinline__ void blc_row_buf(const FwdArgs &a, const float (*w)[W], const float *bias,
                                            float (*hist)[VB / Elem<DT>::bytes], const typename VecIO<VB>::type &X, float m,
                                            __amdgpu_buffer_rsrc_t ro, uint32_t voff, uint32_t soff,
                                            bool keep0 = true, bool keep1 = true, bool keep2 = true)
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
    const bool act = ACT < 0 ? a.act != 0 : ACT != 0;
    const int res = RES < 0 ? a.res_mode : RES;
    const bool eager = EAGER < 0 ? a.eager != 0 : EAGER != 0;
    activate<DT, E>(o, act, eager);
    if (res == CANON_RESIDUAL_UNMASKED || (!MASK && res)) {
#pragma unroll
        for (int e = 0; e < E; ++e) o[e] += xr[e];
    } else if (res == CANON_RESIDUAL_MASKED) {
#pragma unroll
        for (int e = 0; e < E; ++e) o[e] += xm[e];
    }
    BufIO<VB>::template store<store_policy<BIG>()>(VecIO<VB>::template pack<DT>(o), ro, voff, soff);
}

// All rows first .. rows-1 of a slab.
template <int DT, int W, int R, bool MASK, bool BIG, int VB, int ACT, int RES, int EAGER>
__device__ __forceinline__ void blc_rows_buf(const FwdArgs &a, const float (&w)[VB / Elem<DT>::bytes][W], const float (&bias)[VB / Elem<DT>::bytes],
                                             float (&hist)[3][VB / Elem<DT>::bytes], const typename VecIO<VB>::type (&X)[R], const float (&m)[R],
                                             __amdgpu_buffer_rsrc_t ro, uint32_t voff, uint32_t os, int rows)
{
    if (rows == R) {
#pragma unroll
        for (int r = 0; r < R; ++r) blc_row_buf<DT, W, MASK, BIG, VB, ACT, RES, EAGER>(a, w, bias, hist, X[r], m[r], ro, voff, (uint32_t)r * os);
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r)
            if (r < rows) blc_row_buf<DT, W, MASK, BIG, VB, ACT, RES, EAGER>(a, w, bias, hist, X[r], m[r], ro, voff, (uint32_t)r * os);
    }
}

// ... with activation, residual and rounding mode as compile-time constants for the settings CanonLayer uses
// (no activation; residual added or not; either rounding mode), read from the arguments otherwise.
template <int DT, int W, int R, bool MASK, bool BIG, int VB>
__device__ __forceinline__ void blc_rows_dispatch(const FwdArgs &a, const float (&w)[VB / Elem<DT>::bytes][W], const float (&bias)[VB / Elem<DT>::bytes],
                                                  float (&hist)[3][VB / Elem<DT>::bytes], const typename VecIO<VB>::type (&X)[R], const float (&m)[R],
                                                  __amdgpu_buffer_rsrc_t ro, uint32_t voff, uint32_t os, int rows)
{
    // without a mask both residual modes add the raw input
    const int res = (!MASK && a.res_mode) ? CANON_RESIDUAL_UNMASKED : a.res_mode;
    constexpr int XR = CANON_RESIDUAL_UNMASKED, XM = CANON_RESIDUAL_MASKED, NONE = CANON_RESIDUAL_NONE;
    // (an instance with SiLU and the rounding mode fixed at compile time measured no faster than this one)
    if (a.act) blc_rows_buf<DT, W, R, MASK, BIG, VB, -1, -1, -1>(a, w, bias, hist, X, m, ro, voff, os, rows);
    else if (!a.eager && res == XR) blc_rows_buf<DT, W, R, MASK, BIG, VB, 0, XR, 0>(a, w, bias, hist, X, m, ro, voff, os, rows);
    else if (!a.eager && res == XM) blc_rows_buf<DT, W, R, MASK, BIG, VB, 0, XM, 0>(a, w, bias, hist, X, m, ro, voff, os, rows);
    else if (!a.eager && res == NONE) blc_rows_buf<DT, W, R, MASK, BIG, VB, 0, NONE, 0>(a, w, bias, hist, X, m, ro, voff, os, rows);
    else if (res == XR) blc_rows_buf<DT, W, R, MASK, BIG, VB, 0, XR, 1>(a, w, bias, hist, X, m, ro, voff, os, rows);
    else if (res == XM) blc_rows_buf<DT, W, R, MASK, BIG, VB, 0, XM, 1>(a, w, bias, hist, X, m, ro, voff, os, rows);
    else blc_rows_buf<DT, W, R, MASK, BIG, VB, -1, -1, -1>(a, w, bias, hist, X, m, ro, voff, os, rows);
}

// What a wave needs to request its slab: the plain kernel gets these as leading scalar arguments, which
// arrive in registers with the wave (kernel-argument preload), so the slab is requested before the argument
// block has been read; the other kernels take them from the block.
struct BlcLead {
    const char *x;
    int64_t x_sb;         // elements
    uint32_t xs;          // bytes between rows of x
    uint32_t L, nvec;
};

// A wave's place in the launch and its view of x.
template <int VB> struct BlcWave {
    uint32_t b, lane, wv, wt, wc, cv0, nl, c0, voff, xs;
    int64_t t0;
    int rows;
    bool active;
    __amdgpu_buffer_rsrc_t rx;   // rows t0-3 .. t0+R-1 of the wave's 64 channel vectors
};

// Places the wave in tile (b, ct, tt).  Uses nothing but `h`.
template <int DT, int R, int VB>
__device__ __forceinline__ void blc_place(const BlcLead &h, const uint32_t b, const uint32_t ct, const uint32_t tt, BlcWave<VB> &g)
{
    constexpr int E = VB / Elem<DT>::bytes;
    constexpr int BY = Elem<DT>::bytes;
    constexpr int WT = kBlcWaves, WC = kBlcWC;
    g.b = b;
    g.lane = threadIdx.x & 63u;
    g.wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    g.wt = g.wv / WC;
    g.wc = g.wv - g.wt * WC;
    g.cv0 = (ct * WC + g.wc) * 64u;                               // the wave's first channel vector
    g.t0 = ((int64_t)tt * WT + g.wt) * R;
    const int64_t left = (int64_t)h.L - g.t0;
    const bool idle = g.cv0 >= h.nvec || left <= 0;               // wave uniform: nothing to do but the barrier
    g.rows = idle ? 0 : (left >= R ? R : (int)left);
    g.nl = idle ? 0u : (h.nvec - g.cv0 < 64u ? h.nvec - g.cv0 : 64u);   // lanes that hold channels
    g.active = g.lane < g.nl;
    const uint32_t cvl = g.cv0 + g.lane < h.nvec ? g.cv0 + g.lane : h.nvec - 1u;   // idle lanes shadow the last vector (taps, state)
    g.c0 = cvl * E;
    g.xs = h.xs;
    // One buffer resource per tensor and wave: lanes by vector offset, rows by scalar offset.  The x resource
    // starts three rows early.  Every access the wave issues lies inside the resource (rows past the end of
    // the sequence are not loaded); only lanes without channels are sent out of range, by their vector offset.
    const char *xw = h.x + ((int64_t)b * h.x_sb + (int64_t)g.cv0 * E) * BY + (g.t0 - 3) * (int64_t)h.xs;
    const uint32_t xrec = idle ? 0u : (uint32_t)(R + 2) * h.xs + g.nl * VB;
    g.rx = __builtin_amdgcn_make_buffer_rsrc((void *)xw, 0, (int)xrec, kBufFlags);
    g.voff = g.active ? g.lane * VB : 0x80000000u;
}

// Requests, for the first wave of a tile, the three rows before its slab, and then the wave's slab.  (The history
// rows first: they are hits in the L2 of the block's XCD and come back before the slab, whose loads no longer wait
// in front of them: B 8, C 960 6.7 -> 6.4 us; gate / up as two tensors at B 8 20.7 -> 20.4 us.)
template <int DT, int W, int R, int VB>
__device__ __forceinline__ void blc_request(const BlcLead &h, const BlcWave<VB> &g, typename VecIO<VB>::type (&X)[R],
                                            typename VecIO<VB>::type (&H)[3])
{
#pragma unroll
    for (int j = 0; j < 3; ++j) H[j] = VecIO<VB>::zero();
    if (g.wt == 0 && g.t0 > 0) {
#pragma unroll
        for (int j = 0; j < 3; ++j)
            if (j >= 3 - (W - 1)) H[j] = BufIO<VB>::template load<kAuxPlain>(g.rx, g.voff, (uint32_t)j * h.xs);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        // rows past the end of the sequence: the slab's last row again (loaded, never used)
        const uint32_t rr = r < g.rows ? (uint32_t)r : (g.rows > 0 ? (uint32_t)(g.rows - 1) : 0u);
        X[r] = BufIO<VB>::template load<kAuxStream>(g.rx, g.voff, (rr + 3u) * h.xs);
    }
}

using ArgsHere = ArgsRead<FwdArgs>;
// ... with the two pointers the taps are fetched through, which the plain kernel receives among its leading
// scalars: large launches request the taps BEFORE the slab, from registers, so that they wait neither for the slab
// in front of them in the queue nor for a read of the argument block (a round trip of its own: with the taps
// requested after it, a wave's taps arrived later than its slab)
struct ArgsLate : ArgsToRead<FwdArgs> {
    const void *weight, *bias;
    uint32_t part;   // pair kernel: which of the two tensors the block works on (0 in the plain kernel)
};
// which of a pair's two parts the block works on; part 1 finds its taps, bias, output and states at fixed distances
// from part 0's, whose argument block the launch carries
template <typename ARGS> __device__ __forceinline__ uint32_t pair_part(const ARGS &) { return 0u; }
__device__ __forceinline__ uint32_t pair_part(const ArgsLate &l) { return l.part; }
__device__ __forceinline__ const void *shifted(const void *p, int64_t bytes) { return p ? (const void *)((const char *)p + bytes) : nullptr; }

template <int DT, int W, int R, bool MASK, bool BIG, bool SEQ, int VB, int MODE, typename ARGS>
__device__ __forceinline__ void blc_block_body(const ARGS &args, const BlcLead &h, const uint32_t tb, const uint32_t ct, const uint32_t tt,
                                               typename VecIO<VB>::type (*tail)[3][64],   // LDS: raw last three rows of each wave's slab
                                               uint32_t (*taps_lds)[64 * (VB / 2) * 4 + 64 * kBlcWaves * ((VB / 2 + kBlcWaves - 1) / kBlcWaves)])   // LDS: taps and bias of each channel tile
{
    constexpr int E = VB / Elem<DT>::bytes;
    constexpr int BY = Elem<DT>::bytes;
    constexpr int WDT = MODE == TAPS_WIDE ? CANON_DTYPE_F32 : DT;   // weight type of the straight-line tap modes
    constexpr int WT = kBlcWaves, WC = kBlcWC;
    using V = VecIO<VB>;
    static_assert(R >= 3, "a slab must hold the three rows the next slab needs");
    BlcWave<VB> wave;
    typename V::type X[R], H[3];
    blc_place<DT, R, VB>(h, tb, ct, tt, wave);
    // the slab before the argument block where the block is still to be read; otherwise after the taps, which
    // measured 0.4-0.7 us faster at B 8 than slab first
    constexpr bool kShare = MODE != TAPS_ANY && kBlcWaves > 1;
    constexpr int NW = TapWords<WDT, E>::NW, NB = TapWords<WDT, E>::NB;   // words per lane
    constexpr int PW = NW / WT > 0 ? NW / WT : 1, PB = (NB + WT - 1) / WT;   // words per thread
    static_assert(!kShare || NW % WT == 0, "taps of a lane split evenly over the waves of a tile");
    uint32_t tpw[PW], tpb[PB];
    // The waves that share a channel tile fetch its taps and bias together, each a contiguous WT-th of them, and
    // pass them on through LDS with the hand-over of the slab tails (one barrier for both).
    auto fetch_shared_taps = [&](const void *weight, const void *bias, uint32_t nvec_row) {
        constexpr int WBY = Elem<WDT>::bytes;
        const uint32_t g = wave.wt * 64u + wave.lane;                 // thread within the tile's group of waves
        const uint32_t ctile = wave.cv0 < nvec_row ? wave.cv0 * E : 0u;     // first channel of the tile
        const uint32_t cleft = wave.cv0 < nvec_row ? nvec_row * E - ctile : 0u;
        const uint32_t wbytes = (cleft < 64u * E ? cleft : 64u * E) * 4u * WBY;
        const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc((void *)((const char *)weight + (int64_t)ctile * 4 * WBY), 0, (int)wbytes, kBufFlags);
        const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc((void *)((const char *)(bias ? bias : weight) + (int64_t)ctile * WBY), 0, (int)(wbytes / 4u), kBufFlags);
        buf_load_words<PW>(rw, g * (PW * 4u), tpw);
        // (words past the tile's bias are out of range of the resource and read zero)
        buf_load_words<PB>(rb, g * (PB * 4u) < 64u * NB * 4u ? g * (PB * 4u) : 0x80000000u, tpb);
    };
    // Where the argument block is still to be read the slab is requested ahead of it.  Small launches request the
    // taps last, behind the read of the argument block: every block of the launch reads the same few lines of taps
    // at the same moment, and whatever shares the path to L2 with those loads is late (B 8, C 640 / 960: 5.0 / 6.4 us
    // with the taps last, 5.7 / 7.6 us with the taps at once, before or after the slab).  Large launches request
    // the taps FIRST, through the two addresses among the kernel's leading arguments (B 8 / 32, C 3456: 20.5 -> 19.9
    // / 73.6 -> 72.9 us; with a mask at B 16: 38.2 -> 37.8 us; through two pointers read from the argument segment
    // ahead of the block instead: 20.0 / 73.1 / 38.0 us).
    constexpr bool kTapsFirst = ARGS::kLate && BIG && kShare;
    constexpr int64_t kWBY = Elem<WDT>::bytes;
    const uint32_t part = pair_part(args);
    if constexpr (ARGS::kLate) {
        if constexpr (kTapsFirst)
            fetch_shared_taps(shifted(args.weight, (int64_t)(part * h.nvec) * (E * 4 * kWBY)),
                              shifted(args.bias, (int64_t)(part * h.nvec) * (E * kWBY)), h.nvec);
        blc_request<DT, W, R, VB>(h, wave, X, H);
    }
    const FwdArgs &a = args.get();
    const uint32_t cshift = part ? a.pair_c : 0u;   // the block's channels in tensors that cover both parts of a pair
    const uint32_t b = wave.b, lane = wave.lane, wv = wave.wv, wt = wave.wt, wc = wave.wc, cv0 = wave.cv0, nl = wave.nl, c0 = wave.c0;
    const uint32_t voff = wave.voff, xs = wave.xs;
    const int64_t t0 = wave.t0;
    const int rows = wave.rows;
    const bool active = wave.active;
    const uint32_t os = (uint32_t)(a.o_sl * BY);
    char *ow = a.out + (part ? a.pair_out_shift : 0) + ((int64_t)b * a.o_sb + (int64_t)cv0 * E) * BY + t0 * (int64_t)os;
    // (rows past the end of the sequence are not stored; lanes without channels are out of range)
    const uint32_t orec = rows == 0 ? 0u : (uint32_t)(R - 1) * os + nl * VB;
    const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc((void *)ow, 0, (int)orec, kBufFlags);

    float m[R], mh[3];
    int32_t sq[SEQ ? R + 3 : 1];   // sequence index of rows t0-3 .. t0+R-1
    RawTaps<E> raw;
    TapWords<WDT, E> tw;
    const uint32_t g = wt * 64u + lane;                         // thread within the tile's group of waves
    if constexpr (kShare) {
        if constexpr (!kTapsFirst)
            fetch_shared_taps(shifted(a.weight, (int64_t)cshift * (4 * kWBY)), shifted(a.bias, (int64_t)cshift * kWBY), a.nvec);
    } else if constexpr (MODE != TAPS_ANY) {
        fetch_taps_contiguous<WDT, E>(a.weight, a.bias, c0, tw);
    }
    if constexpr (!ARGS::kLate) blc_request<DT, W, R, VB>(h, wave, X, H);
#pragma unroll
    for (int r = 0; r < R; ++r) m[r] = 0.0f;
#pragma unroll
    for (int j = 0; j < (SEQ ? R + 3 : 1); ++j) sq[j] = 0;
#pragma unroll
    for (int j = 0; j < 3; ++j) mh[j] = 0.0f;
    if (rows > 0) {
        if constexpr (MODE == TAPS_ANY)
            fetch_taps<W, E>(a.weight, a.bias, a.w_sc, a.w_sk, a.w_dtype, a.w_vec != 0, c0, raw);
        if constexpr (SEQ) load_seq_rows_wave<R + 3>(a.seq, (int64_t)b * a.q_sb, t0 - 3, a.L, a.q_sl, lane, sq);
        if constexpr (MASK) {
            // mask of the three rows before the slab and of the slab, last so that nothing is issued after its wait
            float mm[R + 3];
            load_mask_rows_wave<R + 3>(a.mask, (int64_t)b * a.m_sb, t0 - 3, a.L, a.m_sl, a.mask_dtype, lane, mm);
#pragma unroll
            for (int j = 0; j < 3; ++j) mh[j] = mm[j];
#pragma unroll
            for (int r = 0; r < R; ++r) m[r] = mm[3 + r];
        }
    }

    // hand the raw tail of this slab to the wave that owns the next slab of the same channel tile
    if constexpr (WT > 1) {
        if constexpr (kShare) {
            uint32_t *tl = taps_lds[wc];
#pragma unroll
            for (int i = 0; i < PW; ++i) tl[g * PW + i] = tpw[i];
            // every thread stores its bias words, also the threads past the tile's bias (they hold zeros and write
            // behind it, inside the array): under a condition the compiler moves the bias load into the branch,
            // behind the wait for the taps, and the block pays a second memory round trip before its barrier
            static_assert(64 * NW + 64 * WT * PB <= (int)(sizeof(taps_lds[0]) / sizeof(uint32_t)), "bias words of all threads fit the LDS array");
#pragma unroll
            for (int i = 0; i < PB; ++i) tl[64 * NW + g * PB + i] = tpb[i];
        }
#pragma unroll
        for (int j = 0; j < 3; ++j) tail[wv][j][lane] = X[R - 3 + j];
        __syncthreads();
        if (wt > 0) {
#pragma unroll
            for (int j = 0; j < 3; ++j)
                if (j >= 3 - (W - 1)) H[j] = tail[wv - WC][j][lane];
        }
        if constexpr (kShare) {
            const uint32_t *tl = taps_lds[wc];
#pragma unroll
            for (int i = 0; i < NW; ++i) tw.w[i] = tl[lane * NW + i];
#pragma unroll
            for (int i = 0; i < NB; ++i) tw.b[i] = tl[64 * NW + lane * NB + i];
        }
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
                hist[j][e] = load1<DT>(a.init, b * a.i_sb + (int64_t)(cshift + c0 + e) * a.i_sc + (int64_t)(a.S_in - 3 + j) * a.i_ss);
        }
    }
    float w[E][W], bias[E];
    if constexpr (MODE == TAPS_ANY) decode_taps<DT, W, E>(raw, a.w_dtype, a.w_vec != 0, a.bias != nullptr, w, bias);
    else decode_taps_contiguous<DT, WDT, E>(tw, a.bias != nullptr, w, bias);
    if constexpr (SEQ) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (r >= rows) continue;
            // rows t-3, t-2, t-1 count only if they carry the index of row t; sequence boundaries are rare,
            // so the all-kept case takes the plain code
            const int32_t cur = sq[3 + r];
            const bool k0 = sq[r] == cur, k1 = sq[r + 1] == cur, k2 = sq[r + 2] == cur;
            if (k0 && k1 && k2) blc_row_buf<DT, W, MASK, BIG, VB>(a, w, bias, hist, X[r], m[r], ro, voff, (uint32_t)r * os);
            else blc_row_buf<DT, W, MASK, BIG, VB>(a, w, bias, hist, X[r], m[r], ro, voff, (uint32_t)r * os, k0, k1, k2);
        }
    } else {
        blc_rows_dispatch<DT, W, R, MASK, BIG, VB>(a, w, bias, hist, X, m, ro, voff, os, rows);
    }

    if (a.fin && active && t0 + rows == (int64_t)a.L) {
        const char *xb = h.x + ((int64_t)b * h.x_sb + c0) * BY;
        for (int slot = 0; slot < a.S_out; ++slot) {
            const int64_t t = (int64_t)a.L - a.S_out + slot;
            float v[E];
#pragma unroll
            for (int e = 0; e < E; ++e) v[e] = 0.0f;
            if (t >= 0) {
                V::template unpack<DT>(V::template load<false>(xb + t * (int64_t)xs), v);
                if constexpr (MASK) {
                    const float mm = load_mask(a.mask, b * a.m_sb + t * a.m_sl, a.mask_dtype);
#pragma unroll
                    for (int e = 0; e < E; ++e) v[e] = mul_round<DT>(v[e], mm);
                }
            } else if (a.init && a.S_in + t >= 0) {
#pragma unroll
                for (int e = 0; e < E; ++e)
                    v[e] = load1<DT>(a.init, b * a.i_sb + (int64_t)(cshift + c0 + e) * a.i_sc + (a.S_in + t) * a.i_ss);
            }
#pragma unroll
            for (int e = 0; e < E; ++e)
                store1<DT>(a.fin, b * a.f_sb + (int64_t)(cshift + c0 + e) * a.f_sc + slot * a.f_ss, v[e]);
        }
    }
}

// The block's code once per tap layout (wave-uniform choice): the contiguous layouts are straight-line
// loads, the general one branches on the run-time weight type between its loads and waits there.
template <int DT, int W, int R, bool MASK, bool BIG, bool SEQ = false, int VB = kBlcVecBytes, typename ARGS>
__device__ __forceinline__ void blc_block(const ARGS &a, const BlcLead &h, const uint32_t tap_mode, const uint32_t b,
                                          const uint32_t ct, const uint32_t tt)
{
    __shared__ typename VecIO<VB>::type tail[kBlcWaves * kBlcWC][3][64];
    // taps and bias of the block's channel tiles as fetched by its waves together: fp32 weights of 16-bit x are the
    // largest case, 64 lanes x 4 channels x (4 taps + bias) x 4 bytes
    constexpr int kTapWordsLds = 64 * (VB / 2) * 4 + 64 * kBlcWaves * ((VB / 2 + kBlcWaves - 1) / kBlcWaves);
    __shared__ uint32_t taps_lds[kBlcWC][kTapWordsLds];
    if constexpr (W == 4) {
        if (tap_mode == TAPS_SAME) {
            blc_block_body<DT, W, R, MASK, BIG, SEQ, VB, TAPS_SAME>(a, h, b, ct, tt, tail, taps_lds);
            return;
        }
        if constexpr (DT != CANON_DTYPE_F32) {
            if (tap_mode == TAPS_WIDE) {
                blc_block_body<DT, W, R, MASK, BIG, SEQ, VB, TAPS_WIDE>(a, h, b, ct, tt, tail, taps_lds);
                return;
            }
        }
    }
    blc_block_body<DT, W, R, MASK, BIG, SEQ, VB, TAPS_ANY>(a, h, b, ct, tt, tail, taps_lds);
}

// Block -> tile.  Workgroups are dealt to the eight XCDs (each with its own L2) in turn, block i to XCD
// i % 8.  The tiles are numbered so that `chunk` consecutive time tiles of one channel tile follow each
// other on ONE XCD: the three rows of history that the first wave of a tile re-reads were requested by
// the tile before it a moment earlier and come out of that L2 instead of memory.  The columns
// q = (b * ngroups + tg) * nct + ct (tg: a group of `chunk` time tiles) are dealt to the XCDs in turn,
// so the launch still sweeps memory in address order.
//
// ... with the blocks numbered in one dimension (block = (column group * chunk + tile of the group) * 8 + XCD)
template <int DT, int W, int R, bool MASK, bool BIG, bool SEQ = false, int VB = kBlcVecBytes>
__device__ __forceinline__ void blc_block_linear(const FwdArgs &a, const uint32_t blk)
{
    const uint32_t jq = blk >> 3;
    const uint32_t jg = fdiv(jq, a.div_nseg);
    const uint32_t q = jg * 8u + (blk & 7u);
    if (q >= a.ntasks) return;   // whole block, before the barrier
    const uint32_t qr = fdiv(q, a.div_nct);
    const uint32_t ct = q - qr * a.nct;
    const uint32_t b = fdiv(qr, a.div_ntt);
    const uint32_t tt = (qr - b * a.nseg) * a.chunk + (jq - jg * a.chunk);
    if (tt >= a.ntt) return;
    const BlcLead h = {a.x, a.x_sb, (uint32_t)(a.x_sl * Elem<DT>::bytes), a.L, a.nvec};
    blc_block<DT, W, R, MASK, BIG, SEQ, VB>(ArgsHere{a}, h, (uint32_t)a.tap_mode, b, ct, tt);
}

// ... and the same in the plain kernel from leading scalar arguments: fourteen dwords, the most that arrive in
// registers.  CANON_BLC_LEAD lists them once, for the kernel's signature and for the struct that mirrors the
// kernel-argument segment (the argument block behind them is read through its offset in that struct).
//   x_sbv    batch stride of x in lane vectors (kBlcVecBytes)
//   packed   log2(chunk) | tap mode << 2 | s1 << 4 | s2 << 5 of the division by nct | s1 << 10 | s2 << 11 of that
//            by ngroups | nct << 16 (the planner keeps nct below 2^16 and chunk a power of two)
//   w_lo, b_lo, wb_hi   weight and bias addresses: low words, and the two high words' low halves (device addresses
//            have 48 bits; checked on the host).  With them in registers the taps are requested without a read of
//            the argument block in front of them.
#define CANON_BLC_LEAD(X)                                                                                              \
    X(const char *, x) X(uint32_t, x_sbv) X(uint32_t, xs) X(uint32_t, L) X(uint32_t, nvec) X(uint32_t, ncols)        \
    X(uint32_t, nct_m) X(uint32_t, ngroups) X(uint32_t, ngroups_m) X(uint32_t, packed) X(uint32_t, w_lo)             \
    X(uint32_t, b_lo) X(uint32_t, wb_hi)
struct BlcSegment {
    CANON_BLC_LEAD(CANON_LEAD_FIELD)
    FwdArgs a;
};
static_assert(offsetof(BlcSegment, a) == 14 * 4, "fourteen leading dwords, then the argument block");

template <int DT, int W, int R, bool MASK, bool BIG>
__global__ __launch_bounds__(kBlcThreads) void canon_fwd_blc_kernel(CANON_BLC_LEAD(CANON_LEAD_PARAM) const FwdArgs a)
{
    const uint32_t lg = packed & 3u, nct = packed >> 16;
    const uint32_t jq = blockIdx.x >> 3;
    const uint32_t jg = jq >> lg;
    const uint32_t q = jg * 8u + (blockIdx.x & 7u);
    if (q >= ncols) return;   // whole block, before the barrier
    const uint32_t qr = fdiv(q, FastDiv{nct, nct_m, (packed >> 4) & 1u, (packed >> 5) & 31u});
    const uint32_t ct = q - qr * nct;
    const uint32_t b = fdiv(qr, FastDiv{ngroups, ngroups_m, (packed >> 10) & 1u, (packed >> 11) & 31u});
    const uint32_t tt = ((qr - b * ngroups) << lg) + (jq - (jg << lg));
    if ((uint64_t)tt * (kBlcWaves * R) >= L) return;   // past the last time tile
    const BlcLead h = {x, (int64_t)x_sbv * (kBlcVecBytes / Elem<DT>::bytes), xs, L, nvec};
#ifdef CANON_NO_LATE_ARGS
    // build switch: the argument block read the ordinary way, at the top of the kernel (for a toolchain whose
    // kernel-argument segment is not laid out like BlcSegment: costs speed, not correctness)
    blc_block<DT, W, R, MASK, BIG>(ArgsHere{a}, h, (packed >> 2) & 3u, b, ct, tt);
    return;
#endif
    ArgsLate late;
    late.offset = (uint32_t)offsetof(BlcSegment, a);
    late.weight = (const void *)((uint64_t)w_lo | (uint64_t)(wb_hi & 0xFFFFu) << 32);
    late.bias = (const void *)((uint64_t)b_lo | (uint64_t)(wb_hi >> 16) << 32);
    late.part = 0u;
    blc_block<DT, W, R, MASK, BIG>(late, h, (packed >> 2) & 3u, b, ct, tt);
}

// Two tensors of the same shape, each dense ([B, L, C] with nothing between rows or sequences), in ONE launch of the
// plain kernel's code: Canon-D's gate and up where they are.  The columns of part 1 follow those of part 0; a block
// picks its tensor from two leading pointers, and the row and batch strides, which the plain kernel receives,
// follow from nvec and L.  `a` is part 0's argument block; part 1's taps, bias, output and states lie at the
// distances a.pair_c / a.pair_out_shift from part 0's (see blc_block_body).  Only for taps the straight-line
// modes cover (the planner sees to that), and not in a build with -DCANON_NO_LATE_ARGS, which plans no such launch.
#ifndef CANON_NO_LATE_ARGS
#define CANON_BLC_PAIR_LEAD(X)                                                                                         \
    X(const char *, x0) X(const char *, x1) X(uint32_t, L) X(uint32_t, nvec) X(uint32_t, ncols) X(uint32_t, nct_m)     \
    X(uint32_t, ngroups) X(uint32_t, ngroups_m) X(uint32_t, packed) X(uint32_t, w_lo) X(uint32_t, b_lo) X(uint32_t, wb_hi)
struct BlcPairSegment {
    CANON_BLC_PAIR_LEAD(CANON_LEAD_FIELD)
    FwdArgs a;
};
static_assert(offsetof(BlcPairSegment, a) == 14 * 4, "fourteen leading dwords, then the argument block");

template <int DT, int W, int R, bool MASK, bool BIG>
__global__ __launch_bounds__(kBlcThreads) void canon_fwd_blc_pair_kernel(CANON_BLC_PAIR_LEAD(CANON_LEAD_PARAM) const FwdArgs a)
{
    const uint32_t lg = packed & 3u, nct = packed >> 16;
    const uint32_t jq = blockIdx.x >> 3;
    const uint32_t jg = jq >> lg;
    uint32_t q = jg * 8u + (blockIdx.x & 7u);
    if (q >= 2u * ncols) return;   // whole block, before the barrier
    const uint32_t part = q >= ncols ? 1u : 0u;
    q -= part * ncols;
    const uint32_t qr = fdiv(q, FastDiv{nct, nct_m, (packed >> 4) & 1u, (packed >> 5) & 31u});
    const uint32_t ct = q - qr * nct;
    const uint32_t b = fdiv(qr, FastDiv{ngroups, ngroups_m, (packed >> 10) & 1u, (packed >> 11) & 31u});
    const uint32_t tt = ((qr - b * ngroups) << lg) + (jq - (jg << lg));
    if ((uint64_t)tt * (kBlcWaves * R) >= L) return;   // past the last time tile
    const BlcLead h = {part ? x1 : x0, (int64_t)L * nvec * (kBlcVecBytes / Elem<DT>::bytes), nvec * (uint32_t)kBlcVecBytes, L, nvec};
    ArgsLate late;
    late.offset = (uint32_t)offsetof(BlcPairSegment, a);
    late.weight = (const void *)((uint64_t)w_lo | (uint64_t)(wb_hi & 0xFFFFu) << 32);
    late.bias = (const void *)((uint64_t)b_lo | (uint64_t)(wb_hi >> 16) << 32);
    late.part = part;
    blc_block<DT, W, R, MASK, BIG>(late, h, (packed >> 2) & 3u, b, ct, tt);
}
#endif  // CANON_NO_LATE_ARGS

// the same over packed variable-length sequences (seq_idx)
template <int DT, int W, int R, bool MASK>
__global__ __launch_bounds__(kBlcThreads) void canon_fwd_blc_seq_kernel(const FwdArgs a)
{
    blc_block_linear<DT, W, R, MASK, false, true, kBlcVecBytes>(a, blockIdx.x);
}

// fb1..fb3: the first blocks of parts 1..3 once more as leading scalars, which arrive in registers with the wave:
// the block knows its part at once and reads that part's arguments in one round instead of two.
template <int DT, int W, int R, bool MASK, bool BIG>
__global__ __launch_bounds__(kBlcThreads) void canon_fwd_blc_parts_kernel(uint32_t fb1, uint32_t fb2, uint32_t fb3,
                                                                          const PartTable<FwdArgs> m)
{
    const uint32_t blk = blockIdx.x;
    const uint32_t p = (blk >= fb1 ? 1u : 0u) + (blk >= fb2 ? 1u : 0u) + (blk >= fb3 ? 1u : 0u);
    const uint32_t first = p == 0 ? 0u : (p == 1 ? fb1 : (p == 2 ? fb2 : fb3));
    // a copy: its loads are issued together here, not one round after the other where the fields are used
    const FwdArgs a = m.part[p];
    blc_block_linear<DT, W, R, MASK, BIG>(a, blk - first);
}

// ---------------------------------------------------------------------------
// prefill, any strides / any length / either rounding mode: one thread per
// (b, c, chunk of time steps), scalar accesses.  STEPWISE: the chunk is walked
// step by step (time-contiguous rows); otherwise everything it reads is
// requested at once.  Two instances because the second needs twice the
// registers, which costs the first its occupancy.
// ---------------------------------------------------------------------------
template <int DT, bool STEPWISE>
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

    const int32_t *seq = a.seq ? a.seq + (int64_t)b * a.q_sb : nullptr;
    if constexpr (STEPWISE) {
        // time-contiguous rows: step by step (a thread's steps are adjacent bytes, the loads after the first
        // hit the cache; requesting the chunk at once, as below, measured 15 % slower here)
        float h[3] = {0, 0, 0};
        int32_t qh[3] = {0, 0, 0};   // with seq_idx: the sequence each history position belongs to
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
            store1<DT>(a.out, oo + t * a.o_sl, finish<DT>(acc, a.act, a.res_mode, a.eager, xm, xr));
            h[0] = h[1];
            h[1] = h[2];
            h[2] = xm;
        }
    } else {
        // Everything the chunk reads is requested before anything is computed (positions past the end are
        // clamped to the last one and never used): stepping through the chunk with a load, a wait and a store per
        // time step costs one memory round trip per step, because the loads cannot be moved above the stores.
        constexpr int N = (int)kGenericChunk, NH = N + 3;        // the chunk and the three steps before it
        const int64_t last = (int64_t)a.L - 1;
        float xr[NH], mk[NH];
        int32_t sq[NH];
        int64_t tpos[NH];
#pragma unroll
        for (int j = 0; j < NH; ++j) {
            const int64_t t = t_begin - 3 + j;
            tpos[j] = t < 0 ? 0 : (t > last ? last : t);
            xr[j] = load1<DT>(a.x, xo + tpos[j] * a.x_sl);
            mk[j] = 1.0f;
            sq[j] = 0;
        }
        if (seq) {
#pragma unroll
            for (int j = 0; j < NH; ++j) sq[j] = seq[tpos[j] * a.q_sl];
        }
        if (a.mask) {
            int64_t idx[NH];
#pragma unroll
            for (int j = 0; j < NH; ++j) idx[j] = (int64_t)b * a.m_sb + tpos[j] * a.m_sl;
            load_mask_entries<NH, false>(a.mask, 0, idx, a.mask_dtype, mk);
        }
        // masked inputs; before the start of the sequence: the initial state, or zero
        float xm[NH];
#pragma unroll
        for (int j = 0; j < NH; ++j) {
            const int64_t t = t_begin - 3 + j;
            xm[j] = a.mask ? mul_round<DT>(xr[j], mk[j]) : xr[j];
            if (t < 0) {
                xm[j] = 0.0f;
                if (j >= 4 - W && a.init && a.S_in + t >= 0)
                    xm[j] = load1<DT>(a.init, b * a.i_sb + c * a.i_sc + (a.S_in + t) * a.i_ss);
            }
        }
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const int64_t t = t_begin + j;
            if (t >= t_end) break;
            const float x0 = xm[j], x1 = xm[j + 1], x2 = xm[j + 2], x3 = xm[j + 3];   // steps t-3 .. t
            float acc = bv;
            if (seq) {
                // inputs of another packed sequence enter as zeros (neither do positions before the start count:
                // they carry no index of their own and the call has no initial state with seq_idx)
                const int32_t qt = sq[j + 3];
                if (W == 4) acc = fmaf(w[0], (t >= 3 && sq[j] == qt) ? x0 : 0.0f, acc);
                if (W >= 3) acc = fmaf(w[1], (t >= 2 && sq[j + 1] == qt) ? x1 : 0.0f, acc);
                acc = fmaf(w[2], (t >= 1 && sq[j + 2] == qt) ? x2 : 0.0f, acc);
                acc = fmaf(w[3], x3, acc);
            } else {
                if (W == 4) acc = fmaf(w[0], x0, acc);
                if (W >= 3) acc = fmaf(w[1], x1, acc);
                acc = fmaf(w[2], x2, acc);
                acc = fmaf(w[3], x3, acc);
            }
            store1<DT>(a.out, oo + t * a.o_sl, finish<DT>(acc, a.act, a.res_mode, a.eager, x3, xr[j + 3]));
        }
    }
    if (a.fin && ch == a.nseg - 1)
        for (int slot = 0; slot < a.S_out; ++slot) capture_row_state<DT>(a, b, c, slot);
}

// ---------------------------------------------------------------------------
// launch: pick the template instance for a plan
// ---------------------------------------------------------------------------
namespace {

template <int DT, int W, bool MASK, bool BIG, bool EDGE> void launch_bcl_e(const FwdPlan &pl, hipStream_t s)
{
    const FwdArgs &a = pl.args;
    const uint32_t wpb = pl.wpb;
    const dim3 g(pl.grid), b(64 * wpb);
    switch (pl.U) {
#define CANON_BCL_LAUNCH(UU)                                                                                             \
    hipLaunchKernelGGL((canon_fwd_bcl_kernel<DT, W, UU, MASK, BIG, EDGE>), g, b, 0, s, a.x, a.x_sb, a.x_sc, a.ntasks, a.nseg, \
                       a.C, a.div_C.m, a.div_C.s1, a.div_C.s2, a.nvec, wpb, a)
    case 4: CANON_BCL_LAUNCH(4); break;
    case 2: CANON_BCL_LAUNCH(2); break;
    default: CANON_BCL_LAUNCH(1); break;
#undef CANON_BCL_LAUNCH
    }
}

template <int DT, int W, bool MASK, bool BIG> void launch_bcl(const FwdPlan &pl, hipStream_t s)
{
    if (pl.edge) launch_bcl_e<DT, W, MASK, BIG, true>(pl, s);
    else launch_bcl_e<DT, W, MASK, BIG, false>(pl, s);
}

template <int DT, int W, bool MASK, bool BIG> void launch_fwd_vec(const FwdPlan &pl, hipStream_t s)
{
    if (pl.kind == FWD_BCL_SHORT) hipLaunchKernelGGL((canon_fwd_bcl_short_kernel<DT, W, MASK>), dim3(pl.grid), dim3(256), 0, s, pl.args);
    else if (pl.kind == FWD_BCL) launch_bcl<DT, W, MASK, BIG>(pl, s);
    else {
        const FwdArgs &a = pl.args;
        uint32_t lg = 0;
        while ((1u << lg) < a.chunk) ++lg;
        const uint32_t packed = lg | (uint32_t)a.tap_mode << 2 | a.div_nct.s1 << 4 | a.div_nct.s2 << 5 | a.div_ntt.s1 << 10 |
                                a.div_ntt.s2 << 11 | a.nct << 16;
        const uint64_t wp = (uint64_t)(uintptr_t)a.weight, bp = (uint64_t)(uintptr_t)a.bias;
#define CANON_BLC_LAUNCH(RR)                                                                                             \
    hipLaunchKernelGGL((canon_fwd_blc_kernel<DT, W, RR, MASK, BIG>), dim3(pl.grid), dim3(kBlcThreads), 0, s, a.x,        \
                       (uint32_t)(a.x_sb / (kBlcVecBytes / Elem<DT>::bytes)), (uint32_t)(a.x_sl * Elem<DT>::bytes), a.L, a.nvec, \
                       a.ntasks, a.div_nct.m, a.nseg, a.div_ntt.m, packed, (uint32_t)wp, (uint32_t)bp,                 \
                       (uint32_t)(wp >> 32) | (uint32_t)(bp >> 32) << 16, a)
        // (short slabs are planned for unmasked width-4 launches only)
        if constexpr (W == 4 && !MASK) {
            if (pl.rows == kBlcRowsShort) {
                CANON_BLC_LAUNCH(kBlcRowsShort);
                return;
            }
        }
        CANON_BLC_LAUNCH(kBlcRows);
#undef CANON_BLC_LAUNCH
    }
}


template <int DT, int W> void launch_fwd_w(const FwdPlan &pl, hipStream_t s)
{
    const bool mask = pl.args.mask != nullptr;
    if (pl.args.seq) {   // only the channel-contiguous kernel is planned with seq_idx
        if (mask) hipLaunchKernelGGL((canon_fwd_blc_seq_kernel<DT, W, kBlcRows, true>), dim3(pl.grid), dim3(kBlcThreads), 0, s, pl.args);
        else hipLaunchKernelGGL((canon_fwd_blc_seq_kernel<DT, W, kBlcRows, false>), dim3(pl.grid), dim3(kBlcThreads), 0, s, pl.args);
        return;
    }
    // the variants for large launches (stores written through, see store_policy) exist for width 4 only
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
        if (pl.args.x_sl == 1) hipLaunchKernelGGL((canon_fwd_generic_kernel<DT, true>), dim3(pl.grid), dim3(256), 0, s, pl.args);
        else hipLaunchKernelGGL((canon_fwd_generic_kernel<DT, false>), dim3(pl.grid), dim3(256), 0, s, pl.args);
        return;
    }
    switch (pl.args.W) {
    case 2: launch_fwd_w<DT, 2>(pl, s); break;
    case 3: launch_fwd_w<DT, 3>(pl, s); break;
    default: launch_fwd_w<DT, 4>(pl, s); break;
    }
}

template <int DT, bool MASK, bool BIG>
void launch_blc_parts(const PartTable<FwdArgs> &m, uint32_t grid, hipStream_t s)
{
    static_assert(kMaxParts == 4, "the parts kernel takes three first-block scalars");
    hipLaunchKernelGGL((canon_fwd_blc_parts_kernel<DT, 4, kBlcRows, MASK, BIG>), dim3(grid), dim3(kBlcThreads), 0, s,
                       m.first_block[1], m.first_block[2], m.first_block[3], m);
}

#ifndef CANON_NO_LATE_ARGS
template <int DT, bool MASK, bool BIG> void launch_blc_pair(const FwdPartsPlan &pp, hipStream_t s)
{
    FwdArgs a = pp.part[0].args;
    a.pair_out_shift = (int64_t)((intptr_t)pp.part[1].args.out - (intptr_t)pp.part[0].args.out);
    a.pair_c = a.C;
    uint32_t lg = 0;
    while ((1u << lg) < a.chunk) ++lg;
    const uint32_t packed = lg | (uint32_t)a.tap_mode << 2 | a.div_nct.s1 << 4 | a.div_nct.s2 << 5 | a.div_ntt.s1 << 10 |
                            a.div_ntt.s2 << 11 | a.nct << 16;
    const uint64_t wp = (uint64_t)(uintptr_t)a.weight, bp = (uint64_t)(uintptr_t)a.bias;
#define CANON_PAIR_LAUNCH(RR)                                                                                            \
    hipLaunchKernelGGL((canon_fwd_blc_pair_kernel<DT, 4, RR, MASK, BIG>), dim3(pp.grid), dim3(kBlcThreads), 0, s, a.x,   \
                       pp.part[1].args.x, a.L, a.nvec, a.ntasks, a.div_nct.m, a.nseg, a.div_ntt.m, packed, (uint32_t)wp, \
                       (uint32_t)bp, (uint32_t)(wp >> 32) | (uint32_t)(bp >> 32) << 16, a)
    if constexpr (!MASK) {
        if (pp.part[0].rows == kBlcRowsShort) {
            CANON_PAIR_LAUNCH(kBlcRowsShort);
            return;
        }
    }
    CANON_PAIR_LAUNCH(kBlcRows);
#undef CANON_PAIR_LAUNCH
}
#endif

template <int DT> void launch_fwd_parts_t(const FwdPartsPlan &pp, hipStream_t s)
{
#ifndef CANON_NO_LATE_ARGS
    if (pp.pair) {
        const bool mask = pp.part[0].args.mask != nullptr, nt = pp.part[0].args.nt != 0;
        if (mask) {
            if (nt) launch_blc_pair<DT, true, true>(pp, s);
            else launch_blc_pair<DT, true, false>(pp, s);
        } else {
            if (nt) launch_blc_pair<DT, false, true>(pp, s);
            else launch_blc_pair<DT, false, false>(pp, s);
        }
        return;
    }
#endif
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

}  // namespace

// Asking for a kernel's attributes makes the runtime load this file's code object onto the current device.
hipError_t preload_fwd()
{
    hipFuncAttributes attr;
    return hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(&(canon_fwd_generic_kernel<CANON_DTYPE_F32, true>)));
}

void launch_fwd(const FwdPlan &pl, int x_dtype, hipStream_t s)
{
    switch (x_dtype) {
    case CANON_DTYPE_F32: launch_fwd<CANON_DTYPE_F32>(pl, s); break;
    case CANON_DTYPE_BF16: launch_fwd<CANON_DTYPE_BF16>(pl, s); break;
    default: launch_fwd<CANON_DTYPE_F16>(pl, s); break;
    }
}

void launch_fwd_parts(const FwdPartsPlan &pp, int x_dtype, hipStream_t s)
{
    switch (x_dtype) {
    case CANON_DTYPE_F32: launch_fwd_parts_t<CANON_DTYPE_F32>(pp, s); break;
    case CANON_DTYPE_BF16: launch_fwd_parts_t<CANON_DTYPE_BF16>(pp, s); break;
    default: launch_fwd_parts_t<CANON_DTYPE_F16>(pp, s); break;
    }
}

}  // namespace canon
