// libcanon_conv1d.so, host side: argument validation, choice of kernel family
// and launch geometry (the plan), and the extern "C" entry points declared in
// include/canon_conv1d.h.  No kernels in this file; the only device object is
// the static scratch array of canon_conv1d_bwd_static.
#include <stdarg.h>
#include <mutex>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "canon_plan.h"

using namespace canon;

namespace {

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

// tap layout the channel-contiguous kernels can read with straight-line loads (see TapMode)
int tap_mode_of(bool w_vec, const void *bias, int x_dtype, int w_dtype)
{
    if (!w_vec || ((uintptr_t)bias & 3u) != 0) return TAPS_ANY;
    if (w_dtype == x_dtype) return TAPS_SAME;
    return w_dtype == CANON_DTYPE_F32 ? TAPS_WIDE : TAPS_ANY;
}

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

// Byte range [lo, hi) that a [B, C, L] tensor with these element strides touches, and whether it fills it.
struct Extent {
    uintptr_t lo, hi;
    bool dense;
};

Extent extent_of(const void *base, int64_t B, int64_t C, int64_t L, int64_t sb, int64_t sc, int64_t sl, int bytes)
{
    int64_t lo = 0, hi = 0;   // smallest / largest element offset
    const int64_t n[3] = {B - 1, C - 1, L - 1}, s[3] = {sb, sc, sl};
    for (int i = 0; i < 3; ++i) {
        if (s[i] < 0) lo += n[i] * s[i];
        else hi += n[i] * s[i];
    }
    Extent e;
    e.lo = (uintptr_t)base + (uintptr_t)(lo * bytes);
    e.hi = (uintptr_t)base + (uintptr_t)((hi + 1) * bytes);
    e.dense = hi - lo + 1 == B * C * L;
    return e;
}

// Time steps per wave of the channel-contiguous prefill for a problem that moves `bytes` (see kBlcRowsShort).
static int blc_rows_for(const canon_conv1d_fwd_params *p, uint64_t bytes)
{
    return (!p->mask && !p->seq_idx && p->width == 4 && bytes >= kBlcShortSlabBytes) ? kBlcRowsShort : kBlcRows;
}

// blc_rows: time steps per wave of the channel-contiguous kernel; 0 = chosen here from the call's own size
int plan_fwd(const canon_conv1d_fwd_params *p, FwdPlan *plan, int blc_rows = 0)
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
        // Overlapping byte ranges: an output element would overwrite an input another thread still has to read.
        // (Two views that both leave holes may interleave in one buffer without sharing an element; that case is
        // left to the caller.)
        const int xb = elem_bytes(p->x_dtype);
        const Extent ex = extent_of(p->x, p->batch, p->channels, p->seqlen, p->x_stride_b, p->x_stride_c, p->x_stride_l, xb);
        const Extent eo = extent_of(p->out, p->batch, p->channels, p->seqlen, p->out_stride_b, p->out_stride_c, p->out_stride_l, xb);
        if (ex.lo < eo.hi && eo.lo < ex.hi && (ex.dense || eo.dense))
            return fail(CANON_ERR_INVALID_ARGUMENT, "out must not alias x: their memory ranges overlap");
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
    a.tap_mode = tap_mode_of(a.w_vec != 0, p->bias, p->x_dtype, p->w_dtype);
    a.m_vec = mask_run_aligned(p->mask, p->mask_dtype, p->mask_stride_b, p->mask_stride_l, p->x_dtype);
    a.b_pair = p->bias && ((uintptr_t)p->bias & 3u) == 0 && (p->w_dtype == CANON_DTYPE_F32 || p->channels % 2 == 0);
    plan->U = 1;
    plan->edge = false;
    plan->wpb = 4;
    plan->grid = 0;
    plan->kind = FWD_GENERIC;
    if (empty) return CANON_OK;

    const int E = 16 / elem_bytes(p->x_dtype);
    const uint64_t rows = (uint64_t)a.B * a.C;
    a.nt = 2 * rows * a.L * elem_bytes(p->x_dtype) >= kStreamBytes;
    const bool ptr_ok = aligned16(p->x) && aligned16(p->out);
    // packed sequences: the channel-contiguous kernel has a variant (the index is uniform per time row);
    // time-contiguous rows take the strided kernel
    // shorter rows leave most of a wave idle: measured slower than the strided kernel below 16 vectors
    const uint32_t kBclMinVectors = 16;
    const bool bcl_rows = !p->seq_idx && ptr_ok && a.x_sl == 1 && a.o_sl == 1 && a.L / E >= kBclMinVectors;
    // every row starts on a 16-byte boundary and is a whole number of vectors ...
    const bool bcl_aligned = a.L % E == 0 && a.x_sb % E == 0 && a.x_sc % E == 0 && a.o_sb % E == 0 && a.o_sc % E == 0;
    // ... or x and out share one geometry, so that a row is misaligned by the same amount in both
    const bool bcl_edge = !bcl_aligned && a.x_sb == a.o_sb && a.x_sc == a.o_sc && a.x_sb >= 0 && a.x_sc >= 0;
    const bool bcl_ok = bcl_rows && (bcl_aligned || bcl_edge);
    const uint32_t EB = kBlcVecBytes / elem_bytes(p->x_dtype);   // channels per lane of the channel-contiguous kernel
    const bool ptr8_ok = (((uintptr_t)p->x | (uintptr_t)p->out) & (kBlcVecBytes - 1)) == 0;
    const bool blc_ok = ptr8_ok && a.x_sc == 1 && a.o_sc == 1 && a.C % EB == 0 &&
                        a.x_sb % EB == 0 && a.x_sl % EB == 0 && a.o_sb % EB == 0 && a.o_sl % EB == 0 &&
                        a.x_sl != 1 &&
                        // the plain kernel receives the batch stride in lane vectors, the tile count in sixteen bits and
                        // the tap addresses in 48 bits among its leading scalar arguments
                        a.x_sb >= 0 && (uint64_t)(a.x_sb / EB) < (1ull << 32) && (a.C / EB + 63) / 64 < (1u << 16) &&
                        (((uintptr_t)p->weight | (uintptr_t)p->bias) >> 48) == 0 &&
                        // rows are addressed by 32-bit scalar offsets inside a wave's buffer resource
                        a.x_sl > 0 && a.o_sl > 0 &&
                        (uint64_t)(kBlcRows + 3) * (uint64_t)a.x_sl * elem_bytes(p->x_dtype) + 64 * kBlcVecBytes < (1ull << 31) &&
                        (uint64_t)(kBlcRows + 3) * (uint64_t)a.o_sl * elem_bytes(p->x_dtype) + 64 * kBlcVecBytes < (1ull << 31);

    // Time-contiguous rows of at most 32 whole, aligned vectors share waves (canon_fwd_bcl_short_kernel):
    // measured against one row per wave, the kernel below, 2.3x faster at 16 vectors per row, 1.3x at 32.
    // (Longer rows packed back to back the same way lose to the kernel below even where it leaves half of its
    // lanes idle: 4.4-4.6 against 5.1-5.7 TB/s.)
    const uint32_t kBclShortMaxVectors = 32;
    if (!p->seq_idx && ptr_ok && a.x_sl == 1 && a.o_sl == 1 && bcl_aligned && a.L / E >= 1 &&
        a.L / E <= kBclShortMaxVectors && rows < (1ull << 31)) {
        const uint32_t nvec = a.L / E;
        uint32_t shift = 0;
        while ((1u << shift) < nvec) ++shift;                  // one group of lanes per row: the next power of two
        const uint64_t groups_per_wave = 64u >> shift;
        const uint64_t nwaves = (rows + groups_per_wave - 1) / groups_per_wave;
        plan->kind = FWD_BCL_SHORT;
        a.nvec = nvec; a.nseg = 1u << shift; a.chunk = shift; a.ntasks = (uint32_t)rows;
        a.div_C = make_fastdiv(a.C);
        a.nblocks = (uint32_t)((nwaves + 3) / 4);
        plan->grid = a.nblocks;
        return CANON_OK;
    }
    if (bcl_ok) {
        const uint32_t nvec = a.L / E;
        // vectors per lane (1, 2 or 4): the fewest that reach the smallest number of segments per row while
        // >= 2048 waves stay in flight.  Every segment after a row's first re-reads its three inputs of history
        // from memory after the wave's own loads, a second round trip: rows of 144..192 vectors as three
        // segments of one vector per lane ran at 3.3-4.2 TB/s, as one segment of four (half of those idle) at
        // 5+ TB/s.  Idle lane slots cost next to nothing here.
        int U = 1;
        uint64_t best = (nvec + 63u) / 64u;
        for (int cand = 2; cand <= kBclMaxVectorsPerLane; cand *= 2) {
            const uint64_t nseg = (nvec + 64u * cand - 1) / (64u * cand);
            if (nseg < best && rows * nseg >= 2048) {
                U = cand;
                best = nseg;
            }
        }
        const uint64_t nseg = (nvec + 64u * U - 1) / (64u * U);
        const uint64_t ntasks = rows * nseg;
        if (ntasks < (1ull << 31)) {
            plan->kind = FWD_BCL;
            plan->U = U;
            plan->edge = !bcl_aligned;
            a.nvec = nvec; a.nseg = (uint32_t)nseg; a.ntasks = (uint32_t)ntasks;
            a.div_nseg = make_fastdiv(a.nseg); a.div_C = make_fastdiv(a.C);
                        // (measured at C 3456, L 1024, bf16: unmasked B 8 / 32 in blocks of 8 waves -0.1 / -0.9 us against 4;
            // masked in blocks of 1 wave -0.5 / -0.4 us against 4, in blocks of 8 waves +1.5 / +7 us)
            const uint32_t wpb = a.mask ? 1u : (ntasks >= kBclBigLaunch ? (uint32_t)kBclMaxWaves : 4u);
            plan->wpb = wpb;
            a.nblocks = (uint32_t)((ntasks + wpb - 1) / wpb);
            plan->grid = a.nblocks;
            return CANON_OK;
        }
    }
    if (blc_ok) {
        const uint32_t nvec = a.C / EB;
        const uint32_t nct = (nvec + 64 * kBlcWC - 1) / (64 * kBlcWC);          // channel tiles per row
        if (blc_rows == 0) blc_rows = blc_rows_for(p, 2ull * rows * a.L * elem_bytes(p->x_dtype));
        plan->rows = blc_rows;
        const uint32_t ntt = (a.L + kBlcWaves * blc_rows - 1) / (kBlcWaves * blc_rows);   // time tiles per sequence
        // `group` consecutive time tiles of a channel tile run back to back on one XCD (see blc_block_body): the
        // largest power of two up to kBlcGroup (the kernel divides by it with a shift) that leaves at most an
        // eighth of the block slots of a sequence without a tile (such blocks return at once)
        uint32_t group = kBlcGroup;
        while (group > 1 && (uint64_t)((ntt + group - 1) / group * group - ntt) * 8 > ntt) group /= 2;
        const uint32_t ngroups = (ntt + group - 1) / group;
        const uint64_t ncols = (uint64_t)a.B * ngroups * nct;
        const uint64_t nblocks = (ncols + 7) / 8 * 8 * group;
        if (nblocks < (1ull << 31) - 8) {
            plan->kind = FWD_BLC;
            a.nvec = nvec; a.nct = nct; a.ntt = ntt; a.ntasks = (uint32_t)ncols;
            a.nseg = ngroups; a.chunk = group;
            a.div_nct = make_fastdiv(nct); a.div_ntt = make_fastdiv(ngroups); a.div_nseg = make_fastdiv(group);
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
    if (((uintptr_t)p->cache_seqlens | (uintptr_t)p->conv_state_indices) & 3u)
        return fail(CANON_ERR_INVALID_ARGUMENT, "cache_seqlens and conv_state_indices must be 4-byte aligned");
    if (p->state_rows < 0) return fail(CANON_ERR_INVALID_ARGUMENT, "state_rows %d is negative", p->state_rows);
    if (p->cache_seqlens && p->width - 1 > p->state_len)
        return fail(CANON_ERR_INVALID_ARGUMENT, "state_len %d is shorter than width-1 = %d", p->state_len, p->width - 1);
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
    if (!empty) {
        // The state is rewritten in place while other threads still read the token and write the output: neither
        // may lie inside it.  (With a state pool of unstated size the rows the call touches are not known here.)
        const int xb = elem_bytes(p->x_dtype);
        const int64_t srows = p->conv_state_indices ? p->state_rows : p->batch;
        if (srows > 0) {
            const Extent es = extent_of(p->conv_state, srows, p->channels, p->state_len, p->state_stride_b, p->state_stride_c,
                                        p->state_stride_s, xb);
            const Extent ex = extent_of(p->x, p->batch, p->channels, 1, p->x_stride_b, p->x_stride_c, 0, xb);
            const Extent eo = extent_of(p->out, p->batch, p->channels, 1, p->out_stride_b, p->out_stride_c, 0, xb);
            if ((ex.lo < es.hi && es.lo < ex.hi && (ex.dense || es.dense)) || (eo.lo < es.hi && es.lo < eo.hi && (eo.dense || es.dense)))
                return fail(CANON_ERR_INVALID_ARGUMENT, "x and out must not overlap conv_state, which is updated in place");
        }
    }

    UpdArgs &a = plan->args;
    memset(&a, 0, sizeof(a));
    a.x = (const char *)p->x; a.out = (char *)p->out; a.state = (char *)p->conv_state;
    a.weight = p->weight; a.bias = p->bias; a.tmask = p->token_mask;
    a.seqlens = p->cache_seqlens; a.indices = p->conv_state_indices; a.state_rows = (uint32_t)p->state_rows;
    a.x_sb = p->x_stride_b; a.x_sc = p->x_stride_c; a.o_sb = p->out_stride_b; a.o_sc = p->out_stride_c;
    a.s_sb = p->state_stride_b; a.s_sc = p->state_stride_c; a.s_ss = p->state_stride_s;
    a.w_sc = p->w_stride_c; a.w_sk = p->w_stride_k; a.m_sb = p->mask_stride_b;
    a.B = (uint32_t)p->batch; a.C = (uint32_t)p->channels;
    a.W = p->width; a.S = p->state_len; a.w_dtype = p->w_dtype; a.mask_dtype = p->mask_dtype;
    a.act = p->activation; a.res_mode = p->residual_mode; a.eager = p->round_mode;
    a.w_vec = p->width == 4 && p->w_stride_k == 1 && p->w_stride_c == 4 && aligned16(p->weight);
    a.tap_mode = tap_mode_of(a.w_vec != 0, p->bias, p->x_dtype, p->w_dtype);
    plan->kind = UPD_GENERIC;
    plan->grid = 0;
    if (empty) return CANON_OK;

    const int S = p->state_len;
    const int BY = elem_bytes(p->x_dtype);
    const int E = upd_lane_channels(BY, S);           // channels per lane
    const int XB = E * BY;                            // bytes of x / out per lane (2 or 4)
    const bool vec_ok = !p->cache_seqlens && (S == 3 || S == 4 || S == 8) &&
                        ((uintptr_t)p->x | (uintptr_t)p->out) % XB == 0 && (uintptr_t)p->conv_state % 4 == 0 &&
                        a.x_sc == 1 && a.o_sc == 1 && a.C % E == 0 && a.x_sb * BY % XB == 0 && a.o_sb * BY % XB == 0 &&
                        a.s_ss == 1 && a.s_sc == S && a.s_sb * BY % 4 == 0;
    if (vec_ok) {
        plan->kind = UPD_VEC;
        a.nvec = a.C / E;
        // two batch rows per lane halve the tap loads; with little work, more waves matter more
        a.nb = (S != 8 && (uint64_t)a.nvec * a.B / kUpdNB >= 512 * 64) ? kUpdNB : 1;
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
    canon_conv1d_fwd_params qs[kMaxParts];
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
        rc = plan_fwd(&q, &pp->part[i], kBlcRows);   // (the table-of-parts kernel has the long slabs only)
        if (rc != CANON_OK) return rc;
        qs[i] = q;
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
    pp->pair = false;
#ifndef CANON_NO_LATE_ARGS
    // Two parts of one shape, each dense, their outputs strided alike, taps the straight-line modes cover: one launch of
    // the plain kernel's code over both (canon_fwd_blc_pair_kernel), which starts its loads from leading scalar
    // arguments as the single-tensor launch does (gate / up at B 8, C 2 x 1728: 20.3 us against 20.3 through the table).
    if (pp->single && nparts == 2) {
        const FwdArgs &u = pp->part[0].args, &v = pp->part[1].args;
        const bool dense = u.x_sl == (int64_t)u.C && u.x_sb == (int64_t)u.L * u.C && v.x_sl == (int64_t)v.C && v.x_sb == (int64_t)v.L * v.C;
        const uint64_t ncols2 = 2ull * u.ntasks;
        const uint64_t nblocks = (ncols2 + 7) / 8 * 8 * u.chunk;
        if (u.C == v.C && dense && u.o_sb == v.o_sb && u.o_sl == v.o_sl && u.tap_mode == v.tap_mode && u.tap_mode != TAPS_ANY &&
            (uint64_t)u.nvec * kBlcVecBytes < (1ull << 31) && nblocks < (1ull << 31) - 8) {
            pp->pair = true;
            pp->grid = (uint32_t)nblocks;
            // the slab length is chosen on the whole problem, like the store policy
            const int r = blc_rows_for(p, 2ull * (uint64_t)p->batch * (uint64_t)p->channels * (uint64_t)p->seqlen * xb);
            if (r != kBlcRows) {
                for (int i = 0; i < 2; ++i) {
                    rc = plan_fwd(&qs[i], &pp->part[i], r);
                    if (rc != CANON_OK) return rc;
                    pp->part[i].args.nt = nt;
                }
                const uint64_t nb = (2ull * pp->part[0].args.ntasks + 7) / 8 * 8 * pp->part[0].args.chunk;
                if (pp->part[0].kind != FWD_BLC || pp->part[1].kind != FWD_BLC || nb >= (1ull << 31) - 8)
                    return fail(CANON_ERR_UNSUPPORTED, "internal: the pair launch could not be planned with short slabs");
                pp->grid = (uint32_t)nb;
            }
        }
    }
#endif
    // parts that go out as launches of their own are planned as single tensors are
    if (!pp->single && !pp->pair)
        for (int i = 0; i < nparts; ++i) {
            rc = plan_fwd(&qs[i], &pp->part[i]);
            if (rc != CANON_OK) return rc;
            pp->part[i].args.nt = nt;
        }
    return CANON_OK;
}

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
    pp->single = nparts > 1 && all_vec && p->width == 4 && !p->conv_state_indices && nvec_total > 0;
    pp->grid = 0;
    if (pp->single) {
        // batch rows per lane chosen on the whole token, the same for every part
        const uint32_t nb = (p->state_len != 8 && nvec_total * (uint64_t)p->batch / kUpdNB >= 512 * 64) ? kUpdNB : 1;
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

// ---------------------------------------------------------------------------
// backward: planning and launch
// ---------------------------------------------------------------------------
// check_pointers: the call itself (x, dout, dx, weight, dweight and the workspace must be there).  Without it
// (queries) NULL pointers pass and count as aligned.  force_generic: plan the strided kernel whatever the layout.
int plan_bwd(const canon_conv1d_bwd_params *p, BwdPlan *plan, bool check_pointers, bool force_generic = false)
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
    if (p->seq_idx && ((uintptr_t)p->seq_idx & 3u))
        return fail(CANON_ERR_INVALID_ARGUMENT, "seq_idx must be 4-byte aligned");
    if (p->initial_state && p->seq_idx)
        return fail(CANON_ERR_INVALID_ARGUMENT, "initial_state cannot be combined with seq_idx");
    if (p->initial_state && p->initial_len < p->width - 1)
        return fail(CANON_ERR_INVALID_ARGUMENT, "initial_len %d is shorter than width-1 = %d", p->initial_len, p->width - 1);
    if (p->dinitial_state && !p->initial_state)
        return fail(CANON_ERR_INVALID_ARGUMENT, "dinitial_state needs initial_state");
    if (p->dfinal_state && p->seq_idx)
        return fail(CANON_ERR_INVALID_ARGUMENT, "dfinal_state cannot be combined with seq_idx");
    if (p->dfinal_state && p->final_len < 1)
        return fail(CANON_ERR_INVALID_ARGUMENT, "final_len %d must be at least 1 with dfinal_state", p->final_len);
    const bool empty = p->batch == 0 || p->channels == 0 || p->seqlen == 0;
    if (empty && p->dinitial_state && p->batch > 0 && p->channels > 0)
        return fail(CANON_ERR_UNSUPPORTED, "dinitial_state of an empty input (it is all zeros) is left to the caller");
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
    a.seq = p->seq_idx; a.q_sb = p->seq_stride_b; a.q_sl = p->seq_stride_l;
    a.init = (const char *)p->initial_state; a.dinit = (char *)p->dinitial_state;
    a.i_sb = p->init_stride_b; a.i_sc = p->init_stride_c; a.i_ss = p->init_stride_s;
    a.j_sb = p->dinit_stride_b; a.j_sc = p->dinit_stride_c; a.j_ss = p->dinit_stride_s;
    a.S_in = p->initial_state ? p->initial_len : 0;
    a.dfin = (const char *)p->dfinal_state; a.S_out = p->dfinal_state ? p->final_len : 0;
    a.k_sb = p->dfinal_stride_b; a.k_sc = p->dfinal_stride_c; a.k_ss = p->dfinal_stride_s;
    a.B = (uint32_t)p->batch; a.C = (uint32_t)p->channels; a.L = (uint32_t)p->seqlen;
    a.W = p->width; a.w_dtype = p->w_dtype; a.mask_dtype = p->mask_dtype;
    a.act = p->activation; a.res_mode = p->residual_mode;
    a.w_vec = p->width == 4 && p->w_stride_k == 1 && p->w_stride_c == 4 && aligned16(p->weight);
    plan->kind = BWD_GENERIC;
    plan->U = 1;
    plan->grid = 0;
    plan->workspace_bytes = 0;
    if (empty) return CANON_OK;   // the caller's dweight/dbias are zero filled by canon_conv1d_bwd

    const int E = 16 / elem_bytes(p->x_dtype);
    a.b_pair = p->bias && ((uintptr_t)p->bias & 3u) == 0 && (p->w_dtype == CANON_DTYPE_F32 || p->channels % 2 == 0);
    a.m_vec = mask_run_aligned(p->mask, p->mask_dtype, p->mask_stride_b, p->mask_stride_l, p->x_dtype);
    const bool ptrs16 = aligned16(p->x) && aligned16(p->dout) && aligned16(p->dx);
    // packed sequences: only the walk kernel gates taps by sequence index.  States (the history before t = 0, the
    // gradient of the captured final state): the walk kernel and the channel-contiguous one.
    const bool packed = force_generic || p->seq_idx != nullptr;
    const bool states = p->initial_state != nullptr || p->dfinal_state != nullptr;
    const bool rows = !packed && !states && ptrs16 && a.x_sl == 1 && a.g_sl == 1 && a.d_sl == 1 && a.L % E == 0 && a.L / E >= 16 &&
                      a.x_sb % E == 0 && a.x_sc % E == 0 && a.g_sb % E == 0 && a.g_sc % E == 0 &&
                      a.d_sb % E == 0 && a.d_sc % E == 0 &&
                      // the kernel receives the batch and channel strides of x and dout in vectors, as 32-bit leading scalars
                      a.x_sb >= 0 && a.x_sc >= 0 && a.g_sb >= 0 && a.g_sc >= 0 &&
                      (uint64_t)(a.x_sb / E) < (1ull << 32) && (uint64_t)(a.x_sc / E) < (1ull << 32) &&
                      (uint64_t)(a.g_sb / E) < (1ull << 32) && (uint64_t)(a.g_sc / E) < (1ull << 32);
    if (rows) {
        const uint32_t nvec = a.L / E;
        const uint64_t nrows = (uint64_t)a.B * a.C;
        // vectors per lane: the fewest that reach the smallest number of segments per row (see plan_fwd)
        int U = 1;
        uint64_t best = (nvec + 63u) / 64u;
        for (int cand = 2; cand <= 4; cand *= 2) {
            const uint64_t nseg = (nvec + 64u * cand - 1) / (64u * cand);
            if (nseg < best && nrows * nseg >= 2048) {
                U = cand;
                best = nseg;
            }
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
    // channel-contiguous tensors: a group of kBwdVecBytes of adjacent channels per lane
    const int E8 = kBwdVecBytes / elem_bytes(p->x_dtype);
    const bool ptrs8 = (((uintptr_t)p->x | (uintptr_t)p->dout | (uintptr_t)p->dx) & (uintptr_t)(kBwdVecBytes - 1)) == 0;
    const bool vec = !packed && a.x_sc == 1 && a.g_sc == 1 && a.d_sc == 1 && a.C % E8 == 0 && a.x_sl != 1 &&
                     a.x_sb % E8 == 0 && a.x_sl % E8 == 0 && a.g_sb % E8 == 0 && a.g_sl % E8 == 0 &&
                     a.d_sb % E8 == 0 && a.d_sl % E8 == 0 && ptrs8;
    if (vec) {
        const uint32_t tile = kBwdSlab * kBwdWaves;
        const uint32_t nvec = a.C / E8;
        const uint32_t nct = (nvec + 63) / 64;
        // time steps per block: as long as possible (few partial sets to write and to add up, taps and
        // chunk-end work amortised) while the grid still has one and a half blocks per CU.  The sequence is
        // cut into the fewest equal chunks (whole tiles) that give such a grid: a block walks every tile of
        // its chunk, so chunks of a fixed length would leave the last one mostly empty (L = 520 as 512 + 8).
        const uint32_t max_chunks = (a.L + tile - 1) / tile;   // = tiles per sequence
        uint32_t nchunk = max_chunks, chunk = tile;
        bool found = false;
        for (uint32_t n = 1; n <= max_chunks; ++n) {
            const uint32_t len = ((a.L + n - 1) / n + tile - 1) / tile * tile;
            if (len > (uint32_t)kBwdMaxChunk) continue;
            const uint32_t used = (a.L + len - 1) / len;               // chunks of that length that hold steps
            const bool enough = 2ull * a.B * used * nct >= 256ull * kBwdHalfBlocksPerCU || n == max_chunks;
            if (!found && enough) {
                found = true;
                nchunk = used;
                chunk = len;
                if (max_chunks % used == 0) break;
                continue;
            }
            // the first count that is enough leaves a short last chunk: a slightly larger count that cuts the
            // tiles evenly runs 5-10 % faster (B4 L1024: 8 chunks of 4 tiles 24.9 us, 7 of 5 tiles 27.1 us)
            if (found && (n >= 2 * nchunk || len < 2 * tile)) break;
            if (found && used == n && max_chunks % n == 0) {
                nchunk = used;
                chunk = len;
                break;
            }
        }
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

int plan_update_bwd(const canon_conv1d_update_bwd_params *p, UpdBwdPlan *plan, bool check_pointers)
{
    if (!p) return fail(CANON_ERR_INVALID_ARGUMENT, "params is NULL");
    if (p->struct_size != sizeof(canon_conv1d_update_bwd_params))
        return fail(CANON_ERR_INVALID_ARGUMENT,
                    "struct_size %u does not match this library's canon_conv1d_update_bwd_params (%zu)", p->struct_size,
                    sizeof(canon_conv1d_update_bwd_params));
    if (!valid_dtype(p->x_dtype) || !valid_dtype(p->w_dtype))
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown x_dtype %d or w_dtype %d", p->x_dtype, p->w_dtype);
    if (p->width < CANON_CONV1D_MIN_WIDTH || p->width > CANON_CONV1D_MAX_WIDTH)
        return fail(CANON_ERR_UNSUPPORTED, "width %d not supported (only widths 2..4)", p->width);
    if (p->activation != CANON_ACT_NONE && p->activation != CANON_ACT_SILU)
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown activation %d", p->activation);
    if (p->residual_mode < CANON_RESIDUAL_NONE || p->residual_mode > CANON_RESIDUAL_UNMASKED)
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown residual_mode %d", p->residual_mode);
    if (p->batch < 0 || p->channels < 0)
        return fail(CANON_ERR_INVALID_ARGUMENT, "negative size (batch %lld, channels %lld)", (long long)p->batch,
                    (long long)p->channels);
    if (p->batch >= (1ll << 31) || p->channels >= (1ll << 29) || p->batch * p->channels >= (1ll << 31))
        return fail(CANON_ERR_UNSUPPORTED, "batch*channels must be below 2^31 and channels below 2^29");
    if (p->state_len < 1 || p->state_len < p->width - 1)
        return fail(CANON_ERR_INVALID_ARGUMENT, "state_len %d is shorter than width-1 = %d", p->state_len, p->width - 1);
    if (p->token_mask && !valid_mask_dtype(p->mask_dtype))
        return fail(CANON_ERR_INVALID_ARGUMENT, "unknown mask_dtype %d", p->mask_dtype);
    if (p->dbias && !p->dweight) return fail(CANON_ERR_INVALID_ARGUMENT, "dbias needs dweight");
    if (p->state_rows < 0 || p->state_rows >= (1ll << 31))
        return fail(CANON_ERR_INVALID_ARGUMENT, "state_rows %lld must lie in [0, 2^31)", (long long)p->state_rows);
    if (p->state_rows > 0 && !p->conv_state_indices)
        return fail(CANON_ERR_INVALID_ARGUMENT, "state_rows is the size of the pool conv_state_indices selects from; without them it must be 0");
    const bool empty = p->batch == 0 || p->channels == 0;
    if (check_pointers && !empty) {
        if (!p->x || !p->conv_state || !p->weight || !p->dout || !p->dx)
            return fail(CANON_ERR_INVALID_ARGUMENT, "x, conv_state, weight, dout and dx must not be NULL");
        if (p->dstate && p->dstate == p->dstate_out)
            return fail(CANON_ERR_INVALID_ARGUMENT, "dstate must not alias dstate_out");
    }

    UpdBwdArgs &a = plan->args;
    memset(&a, 0, sizeof(a));
    a.x = (const char *)p->x; a.state = (const char *)p->conv_state; a.dy = (const char *)p->dout;
    a.dso = (const char *)p->dstate_out; a.dx = (char *)p->dx; a.ds = (char *)p->dstate;
    a.weight = p->weight; a.bias = p->bias; a.tmask = p->token_mask;
    a.dweight = p->dweight; a.dbias = p->dbias;
    a.x_sb = p->x_stride_b; a.x_sc = p->x_stride_c; a.g_sb = p->dout_stride_b; a.g_sc = p->dout_stride_c;
    a.d_sb = p->dx_stride_b; a.d_sc = p->dx_stride_c;
    a.s_sb = p->state_stride_b; a.s_sc = p->state_stride_c; a.s_ss = p->state_stride_s;
    a.q_sb = p->dstate_out_stride_b; a.q_sc = p->dstate_out_stride_c; a.q_ss = p->dstate_out_stride_s;
    a.r_sb = p->dstate_stride_b; a.r_sc = p->dstate_stride_c; a.r_ss = p->dstate_stride_s;
    a.w_sc = p->w_stride_c; a.w_sk = p->w_stride_k; a.m_sb = p->mask_stride_b;
    a.B = (uint32_t)p->batch; a.C = (uint32_t)p->channels;
    a.W = p->width; a.S = p->state_len; a.w_dtype = p->w_dtype; a.mask_dtype = p->mask_dtype;
    a.act = p->activation; a.res_mode = p->residual_mode;
    a.seqlens = p->cache_seqlens; a.indices = p->conv_state_indices; a.state_rows = (uint32_t)p->state_rows;
    plan->grid_c = 0;
    plan->workspace_bytes = 0;
    plan->vec = false;
    if (empty) return CANON_OK;

    const int S = p->state_len;
    const int BY = elem_bytes(p->x_dtype);
    const int E = upd_lane_channels(BY, S);
    auto dense_state = [&](const void *ptr, int64_t sb, int64_t sc, int64_t ss) {
        return !ptr || ((uintptr_t)ptr % 4 == 0 && ss == 1 && sc == S && sb * BY % 4 == 0);
    };
    auto dense_token = [&](const void *ptr, int64_t sb, int64_t sc) {
        return (uintptr_t)ptr % 4 == 0 && sc == 1 && sb * BY % 4 == 0;
    };
    // (ring buffer and state pool: the strided kernel)
    plan->vec = !p->cache_seqlens && !p->conv_state_indices && (S == 3 || S == 4) && a.C % E == 0 && (!check_pointers || (
                    dense_token(p->x, a.x_sb, a.x_sc) && dense_token(p->dout, a.g_sb, a.g_sc) &&
                    dense_token(p->dx, a.d_sb, a.d_sc) && dense_state(p->conv_state, a.s_sb, a.s_sc, a.s_ss) &&
                    dense_state(p->dstate_out, a.q_sb, a.q_sc, a.q_ss) && dense_state(p->dstate, a.r_sb, a.r_sc, a.r_ss)));
    // Batch groups.  One channel per thread: enough groups for about four blocks per compute unit, at most 1024.
    // Vector kernel: the four waves of a block split a group, four entries each per round, so a group is 16
    // entries unless that leaves fewer blocks than compute units (measured at B256 C3456 bf16: groups of 16 / 8 / 4
    // entries 8.4 / 9.6 / 13.4 us).  The scratch is sized for whichever needs more, so
    // that its size does not depend on the pointers' alignment.
    const uint32_t cblocks = (a.C + 255u) / 256u;
    uint32_t want = (1024u + cblocks - 1u) / cblocks;
    if (want > 1024u) want = 1024u;
    if (want > a.B) want = a.B;
    const uint32_t group_s = (a.B + want - 1u) / want;
    const uint32_t ngroups_s = (a.B + group_s - 1u) / group_s;
    const uint32_t vblocks = (a.C / E + 63u) / 64u;
    uint32_t group_v = 16u;
    while (group_v > 4u && (uint64_t)vblocks * ((a.B + group_v - 1u) / group_v) < 256u) group_v /= 2u;
    while ((a.B + group_v - 1u) / group_v > 65535u) group_v *= 2u;
    const uint32_t ngroups_v = (a.B + group_v - 1u) / group_v;
    if (plan->vec) {
        a.group = group_v; a.ngroups = ngroups_v; plan->grid_c = vblocks;
    } else {
        a.group = group_s; a.ngroups = ngroups_s; plan->grid_c = cblocks;
    }
    if (a.ngroups > 65535u) return fail(CANON_ERR_UNSUPPORTED, "batch too large for the decode backward");
    if (p->dweight) {
        const uint32_t most = ngroups_v > ngroups_s ? ngroups_v : ngroups_s;
        plan->workspace_bytes = (int64_t)most * a.C * 5 * (int64_t)sizeof(float);
        a.partial = (float *)p->workspace;
        if (check_pointers && (!p->workspace || !aligned16(p->workspace) || p->workspace_bytes < plan->workspace_bytes))
            return fail(CANON_ERR_INVALID_ARGUMENT, "workspace must be 16-byte aligned and at least %lld bytes (got %lld)",
                        (long long)plan->workspace_bytes, (long long)p->workspace_bytes);
    }
    return CANON_OK;
}

int check_launch(const char *what)
{
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(CANON_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return CANON_OK;
}

}  // namespace

#define CANON_API __attribute__((visibility("default")))

extern "C" {

CANON_API int canon_conv1d_abi_version(void) { return CANON_CONV1D_ABI_VERSION; }

CANON_API const char *canon_conv1d_last_error(void) { return g_err; }

CANON_API int canon_conv1d_fwd(const canon_conv1d_fwd_params *p, void *stream)
{
    FwdPlan pl;
    const int rc = plan_fwd(p, &pl);
    if (rc != CANON_OK) return rc;
    if (pl.grid == 0) return CANON_OK;
    hipStream_t s = (hipStream_t)stream;
    launch_fwd(pl, p->x_dtype, s);
    return check_launch("canon_conv1d_fwd");
}

CANON_API int canon_conv1d_update(const canon_conv1d_update_params *p, void *stream)
{
    UpdPlan pl;
    const int rc = plan_update(p, &pl);
    if (rc != CANON_OK) return rc;
    if (pl.grid == 0) return CANON_OK;
    hipStream_t s = (hipStream_t)stream;
    launch_update(pl, p->x_dtype, s);
    return check_launch("canon_conv1d_update");
}

CANON_API int canon_conv1d_bwd(const canon_conv1d_bwd_params *p, void *stream)
{
    BwdPlan pl;
    const int rc = plan_bwd(p, &pl, true);
    if (rc != CANON_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    if (pl.grid == 0) {
        // nothing to sum: the gradients of the parameters are zero
        // (a fill kernel rather than a memset, so that the call can be captured into a HIP graph)
        if (p->channels > 0) {
            launch_zero(p->dweight, (uint32_t)(p->channels * p->width), s);
            if (p->dbias) launch_zero(p->dbias, (uint32_t)p->channels, s);
            return check_launch("canon_conv1d_bwd");
        }
        return CANON_OK;
    }
    launch_bwd(pl, p->x_dtype, s);
    return check_launch("canon_conv1d_bwd");
}

CANON_API int64_t canon_conv1d_bwd_workspace_bytes(const canon_conv1d_bwd_params *p)
{
    BwdPlan pl;
    if (plan_bwd(p, &pl, false) != CANON_OK) return -1;
    int64_t need = pl.workspace_bytes;
    // Which kernel runs depends on the alignment of x, dout and dx as well.  With all three given the answer is that
    // of the call; with one missing it covers the strided kernel too, which a misaligned pointer would select.
    if (!p->x || !p->dout || !p->dx) {
        if (plan_bwd(p, &pl, false, true) != CANON_OK) return -1;
        if (pl.workspace_bytes > need) need = pl.workspace_bytes;
    }
    return need;
}

// The scratch of canon_conv1d_bwd_static: one copy per GPU, at its own address on each.  On the host the
// array's name is only a handle for hipGetSymbolAddress; kernels and fills take the device address it returns.
constexpr int64_t kStaticScratchBytes = CANON_CONV1D_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device address of the current GPU's copy, looked up once per device (by canon_conv1d_init, else by the first
// call of canon_conv1d_bwd_static on that GPU: the lookup makes the runtime load this file's code object, which
// is when the array's memory is allocated).
static int static_scratch(const char *who, void **out)
{
    constexpr int kMaxDevices = 64;
    static void *ptr_of_device[kMaxDevices];
    static std::mutex lookup;
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(CANON_ERR_LAUNCH, "%s: hipGetDevice: %s", who, hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(CANON_ERR_UNSUPPORTED, "%s: device %d", who, dev);
    std::lock_guard<std::mutex> hold(lookup);
    if (!ptr_of_device[dev]) {
        void *q = nullptr;
        e = hipGetSymbolAddress(&q, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !q) return fail(CANON_ERR_LAUNCH, "%s: hipGetSymbolAddress: %s", who, hipGetErrorString(e));
        ptr_of_device[dev] = q;
    }
    *out = ptr_of_device[dev];
    return CANON_OK;
}

CANON_API int canon_conv1d_init(void)
{
    void *ptr;
    const int rc = static_scratch("canon_conv1d_init", &ptr);
    if (rc != CANON_OK) return rc;
    const hipError_t loaded[3] = {preload_fwd(), preload_update(), preload_bwd()};
    for (hipError_t e : loaded)
        if (e != hipSuccess) return fail(CANON_ERR_LAUNCH, "canon_conv1d_init: loading the kernels: %s", hipGetErrorString(e));
    return CANON_OK;
}

CANON_API int canon_conv1d_bwd_static(const canon_conv1d_bwd_params *p, void *stream)
{
    if (!p) return fail(CANON_ERR_INVALID_ARGUMENT, "params is NULL");
    if (p->struct_size != sizeof(canon_conv1d_bwd_params))
        return fail(CANON_ERR_INVALID_ARGUMENT, "struct_size %u does not match this library's canon_conv1d_bwd_params (%zu)",
                    p->struct_size, sizeof(canon_conv1d_bwd_params));
    void *ptr;
    int rc = static_scratch("canon_conv1d_bwd_static", &ptr);
    if (rc != CANON_OK) return rc;
    canon_conv1d_bwd_params q = *p;
    q.workspace = ptr;
    q.workspace_bytes = kStaticScratchBytes;
    BwdPlan pl;
    rc = plan_bwd(&q, &pl, false);
    if (rc != CANON_OK) return rc;
    if (pl.workspace_bytes > kStaticScratchBytes)
        return fail(CANON_ERR_UNSUPPORTED,
                    "canon_conv1d_bwd_static: this problem needs %lld bytes of scratch, the library's static buffer holds %lld; "
                    "use canon_conv1d_bwd with a workspace of the caller's",
                    (long long)pl.workspace_bytes, (long long)kStaticScratchBytes);
    // every partial set the reduction reads is written by this launch first: nothing of an earlier call is read
    return canon_conv1d_bwd(&q, stream);
}

CANON_API int canon_conv1d_update_bwd(const canon_conv1d_update_bwd_params *p, void *stream)
{
    UpdBwdPlan pl;
    const int rc = plan_update_bwd(p, &pl, true);
    if (rc != CANON_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    if (pl.grid_c == 0) {
        // an empty batch: the parameter gradients are zero (fill kernels, so that the call can be captured)
        if (p->channels > 0 && p->dweight) {
            launch_zero(p->dweight, (uint32_t)(p->channels * p->width), s);
            if (p->dbias) launch_zero(p->dbias, (uint32_t)p->channels, s);
            return check_launch("canon_conv1d_update_bwd");
        }
        return CANON_OK;
    }
    launch_update_bwd(pl, p->x_dtype, s);
    return check_launch("canon_conv1d_update_bwd");
}

CANON_API int64_t canon_conv1d_update_bwd_workspace_bytes(const canon_conv1d_update_bwd_params *p)
{
    UpdBwdPlan pl;
    if (plan_update_bwd(p, &pl, false) != CANON_OK) return -1;
    return pl.workspace_bytes;
}

CANON_API const char *canon_conv1d_bwd_plan(const canon_conv1d_bwd_params *p)
{
    BwdPlan pl;
    if (plan_bwd(p, &pl, false) != CANON_OK) return nullptr;
    return pl.kind == BWD_BLC_VEC ? "bwd_blc_vec" : pl.kind == BWD_BCL_VEC ? "bwd_bcl_vec" : "bwd_generic";
}

CANON_API const char *canon_conv1d_fwd_plan(const canon_conv1d_fwd_params *p)
{
    FwdPlan pl;
    if (plan_fwd(p, &pl) != CANON_OK) return nullptr;
    if (pl.kind == FWD_BLC && pl.args.seq) return "blc_vec_seq";
    if (pl.kind == FWD_BCL_SHORT) return "bcl_vec_short";
    return pl.kind == FWD_BCL ? "bcl_vec" : pl.kind == FWD_BLC ? "blc_vec" : "generic";
}

CANON_API int canon_conv1d_fwd_plan_waves(const canon_conv1d_fwd_params *p)
{
    FwdPlan pl;
    if (plan_fwd(p, &pl) != CANON_OK) return -1;
    if (pl.grid == 0) return 0;
    return pl.kind == FWD_BCL ? (int)pl.wpb : 4;
}

CANON_API const char *canon_conv1d_update_plan(const canon_conv1d_update_params *p)
{
    UpdPlan pl;
    if (plan_update(p, &pl) != CANON_OK) return nullptr;
    return pl.kind == UPD_VEC ? "update_vec" : "update_generic";
}

CANON_API int canon_conv1d_fwd_parts(const canon_conv1d_fwd_params *p, const canon_conv1d_part *parts, int32_t nparts, void *stream)
{
    FwdPartsPlan pp;
    const int rc = plan_fwd_parts(p, parts, nparts, &pp);
    if (rc != CANON_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    launch_fwd_parts(pp, p->x_dtype, s);
    return check_launch("canon_conv1d_fwd_parts");
}

CANON_API int canon_conv1d_update_parts(const canon_conv1d_update_params *p, const canon_conv1d_part *parts, int32_t nparts,
                              void *stream)
{
    UpdPartsPlan pp;
    const int rc = plan_update_parts(p, parts, nparts, &pp);
    if (rc != CANON_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    launch_update_parts(pp, p->x_dtype, s);
    return check_launch("canon_conv1d_update_parts");
}

CANON_API const char *canon_conv1d_fwd_parts_plan(const canon_conv1d_fwd_params *p, const canon_conv1d_part *parts, int32_t nparts)
{
    FwdPartsPlan pp;
    if (plan_fwd_parts(p, parts, nparts, &pp) != CANON_OK) return nullptr;
    return pp.pair ? "blc_vec_pair" : pp.single ? "blc_vec_parts" : "per_part";
}

CANON_API const char *canon_conv1d_update_parts_plan(const canon_conv1d_update_params *p, const canon_conv1d_part *parts,
                                           int32_t nparts)
{
    UpdPartsPlan pp;
    if (plan_update_parts(p, parts, nparts, &pp) != CANON_OK) return nullptr;
    return pp.single ? "update_vec_parts" : "per_part";
}

}  // extern "C"
