// Canon causal depthwise conv1d for MI355X (gfx950): backward of the prefill
// (dx, and dweight / dbias through partial sets and a fixed-order reduction).
#include "canon_device.h"

namespace canon {

// ---------------------------------------------------------------------------
// backward of the prefill: dx, and per-chunk partial sums of dweight / dbias
//
// Every kernel of this file writes dx and one entry per channel of a partial
// set, partial[(b * nchunk + chunk) * C + c][5] (w0..w3, bias);
// canon_bwd_reduce_kernel sums the sets in a fixed order.
//
// canon_bwd_walk_kernel, the fallback for layouts without a vector kernel
// (any strides): one lane owns a channel and walks a chunk of time steps from
// its END to its start.  dx[t] needs dz[t .. t+W-1] (the three later steps are
// carried in registers), z[t] needs xm[t-3 .. t] (a sliding window refilled
// with one row per step, fetched R rows ahead).  The three dz values just past
// the chunk are recomputed from memory.
//
// With an initial state (a.init) the rows before t = 0 are its last entries
// instead of zeros: they enter the windows (z and dweight) like any other row,
// and the lane that ends at t = 0 also forms their gradient from the three dz
// values it carries out of the loop.
//
// SEQ (packed sequences): the sequence index of every row travels with it
// (window, carried dz values, look-ahead).  A product of a tap with a row of
// another sequence index is dropped wherever it appears: in z, in dx (the dz
// of a later step of another sequence) and in dweight.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float silu_grad(float z)
{
    const float s = __builtin_amdgcn_rcpf(1.0f + __expf(-z));
    return s * (1.0f + z * (1.0f - s));
}

template <int DT, int W, bool MASK, int R, bool SEQ>
__global__ __launch_bounds__(256) void canon_bwd_walk_kernel(const BwdArgs a)
{
    constexpr int BY = Elem<DT>::bytes;
    constexpr int E = 1;     // channels per lane
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
    fetch_taps<W, E>(a.weight, a.bias, a.w_sc, a.w_sk, a.w_dtype, false, c0, raw);

    // rows t_end-4 .. t_end+2 of xm (window for the last step + the three steps past the chunk)
    float xr7[7][E], m7[7];
#pragma unroll
    for (int j = 0; j < 7; ++j) {
        const int64_t t = t_end - 4 + j;
        const int64_t tc = t < 0 ? 0 : (t > Lm1 ? Lm1 : t);
        xr7[j][0] = load1<DT>(xb + tc * xs, 0);
        m7[j] = 1.0f;
    }
    float g3[3][E];
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        const int64_t t = t_end + j;
        g3[j][0] = load1<DT>(gb + (t > Lm1 ? Lm1 : t) * gs, 0);
    }
    if constexpr (MASK) load_mask_rows<7>(a.mask, (int64_t)b * a.m_sb, t_end - 4, a.L, a.m_sl, a.mask_dtype, m7);
    // rows before t = 0: entries of the initial state (not masked), zeros without one
    const char *ib = a.init ? a.init + ((int64_t)b * a.i_sb + (int64_t)c0 * a.i_sc + (int64_t)a.S_in * a.i_ss) * BY : nullptr;
    const int64_t is = a.i_ss * BY;
    float h7[7] = {0, 0, 0, 0, 0, 0, 0};
    if (ib && t_end < 4) {
#pragma unroll
        for (int j = 0; j < 7; ++j) {
            const int64_t t = t_end - 4 + j;
            if (t < 0 && t >= -(int64_t)a.S_in) h7[j] = load1<DT>(ib + t * is, 0);
        }
    }
    int32_t q7[7] = {0, 0, 0, 0, 0, 0, 0};   // sequence indices of the same seven rows
    if constexpr (SEQ) load_seq_rows<7>(a.seq, (int64_t)b * a.q_sb, t_end - 4, a.L, a.q_sl, q7);

    float w[E][W], bias[E];
    decode_taps<DT, W, E>(raw, a.w_dtype, false, a.bias != nullptr, w, bias);

#pragma unroll
    for (int j = 0; j < 7; ++j) {
        const int64_t t = t_end - 4 + j;
        const bool inside = t >= 0 && t <= Lm1;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float v = MASK ? mul_round<DT>(xr7[j][e], m7[j]) : xr7[j][e];
            xr7[j][e] = inside ? v : (t < 0 ? h7[j] : 0.0f);
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
            for (int k = 0; k < W; ++k) {
                const int row = j + 1 + (4 - W) + k;                                   // xm[t_end+j-(W-1)+k]
                const float v = (!SEQ || q7[row] == q7[j + 4]) ? xr7[row][e] : 0.0f;
                z = fmaf(w[e][k], v, z);
            }
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
    // qw[k]: sequence index of xw[k]'s row; qf[j]: of dzf[j]'s step
    int32_t qw[4] = {q7[0], q7[1], q7[2], q7[3]};
    int32_t qf[3] = {q7[4], q7[5], q7[6]};

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
        float G[R], XN[R], HN[R];
        float mk[R], mn[R];
        int32_t QN[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int64_t t = t_hi - r;
            const int64_t tg = t < 0 ? 0 : t;
            const int64_t tn = t - 4 < 0 ? 0 : t - 4;
            G[r] = load1<DT>(gb + tg * gs, 0);
            XN[r] = load1<DT>(xb + tn * xs, 0);
            HN[r] = (ib && t - 4 < 0 && t - 4 >= -(int64_t)a.S_in) ? load1<DT>(ib + (t - 4) * is, 0) : 0.0f;
            QN[r] = SEQ ? a.seq[(int64_t)b * a.q_sb + tn * a.q_sl] : 0;
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
            g[0] = G[r];
            xn[0] = XN[r];
            // the window as this step sees it: rows of other sequences read as zero
            float xs_[4][E];
#pragma unroll
            for (int k = 0; k < 4; ++k)
#pragma unroll
                for (int e = 0; e < E; ++e) xs_[k][e] = (!SEQ || qw[k] == qw[3]) ? xw[k][e] : 0.0f;
#pragma unroll
            for (int e = 0; e < E; ++e) {
                float z = bias[e];
#pragma unroll
                for (int k = 0; k < W; ++k) z = fmaf(w[e][k], xs_[(4 - W) + k][e], z);
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
                acc = fmaf(w[e][W - 2], (!SEQ || qf[0] == qw[3]) ? dzf[0][e] : 0.0f, acc);
                if constexpr (W >= 3) acc = fmaf(w[e][W - 3], (!SEQ || qf[1] == qw[3]) ? dzf[1][e] : 0.0f, acc);
                if constexpr (W == 4) acc = fmaf(w[e][0], (!SEQ || qf[2] == qw[3]) ? dzf[2][e] : 0.0f, acc);
                o[e] = acc;
#pragma unroll
                for (int k = 0; k < W; ++k) dw[e][k] = fmaf(dz[e], xs_[(4 - W) + k][e], dw[e][k]);
                dbs[e] += dz[e];
                dzf[2][e] = dzf[1][e];
                dzf[1][e] = dzf[0][e];
                dzf[0][e] = dz[e];
            }
            if (a.res_mode == CANON_RESIDUAL_MASKED) {
#pragma unroll
                for (int e = 0; e < E; ++e) o[e] += g[e];
            }
            if (a.dfin && t >= (int64_t)a.L - a.S_out) {
                // this step's masked input was captured into slot t - (L - S_out) of the final state
                o[0] += load1<DT>(a.dfin + ((int64_t)b * a.k_sb + (int64_t)c0 * a.k_sc + (t - ((int64_t)a.L - a.S_out)) * a.k_ss) * BY, 0);
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
                xw[0][e] = has_row ? v : HN[r];
            }
            if constexpr (SEQ) {
                qf[2] = qf[1]; qf[1] = qf[0]; qf[0] = qw[3];
                qw[3] = qw[2]; qw[2] = qw[1]; qw[1] = qw[0]; qw[0] = QN[r];
            }
            store1<DT>(db_ + t * ds, 0, o[0]);
        }
    }

    if (a.dinit && ch == 0) {
        // here dzf[i] = dz[i] (zero past the end of the row).  Entry s is the input at t = s - S_in = -d:
        // its gradient is sum_i w[W-1-d-i] * dz[i] over the taps that exist
        char *jb = a.dinit + ((int64_t)b * a.j_sb + (int64_t)c0 * a.j_sc) * BY;
        for (int s = 0; s < a.S_in; ++s) {
            const int d = a.S_in - s;
            float acc = 0.0f;
#pragma unroll
            for (int i = 0; i < 3; ++i) {
                const int k = W - 1 - d - i;
                if (k >= 0) acc = fmaf(w[0][k], dzf[i][0], acc);
            }
            // a final state longer than the row also captured this entry (input at t = -d) in slot S_out - L - d
            const int64_t slot = (int64_t)a.S_out - (int64_t)a.L - d;
            if (a.dfin && slot >= 0)
                acc += load1<DT>(a.dfin + ((int64_t)b * a.k_sb + (int64_t)c0 * a.k_sc + slot * a.k_ss) * BY, 0);
            store1<DT>(jb + (int64_t)s * a.j_ss * BY, 0, acc);
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
// x and dout are read once and dx is written once: streamed (non-temporal) accesses, as in the forward kernels
// (measured at B 8, C 3456, L 1024, bf16: 40.7 -> 37.8 us channel-contiguous, 33.6 -> 30.9 us time-contiguous).
constexpr bool kBwdStream = true;
using BV = VecIO<kBwdVecBytes>;
using BVT = BV::type;   // a lane's piece of one row
template <int DT> __device__ __forceinline__ void unpack_half(const BVT &v, float *f) { BV::template unpack<DT>(v, f); }
template <int DT> __device__ __forceinline__ BVT pack_half(const float *f) { return BV::template pack<DT>(f); }

// One raw row -> the bits of xm = x * mask in the storage type (zero when the row does not exist)
template <int DT, bool MASK>
__device__ __forceinline__ BVT bwd_mask_row(const BVT &raw, float m, bool exists)
{
    constexpr int E = kBwdVecBytes / Elem<DT>::bytes;
    BVT v = raw;
    if constexpr (MASK) {
      // m is the same for the whole wave and 1 for every valid token of a padded batch: x * 1 is x, bit for bit
      if (m != 1.0f) {
        float f[E];
        unpack_half<DT>(raw, f);
#pragma unroll
        for (int e = 0; e < E; ++e) {
            f[e] *= m;
            if constexpr (DT == CANON_DTYPE_F16) asm volatile("" : "+v"(f[e]));   // see mul_round
        }
        v = pack_half<DT>(f);
      }
    }
    if (!exists) v = BV::zero();
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
// after the slab.  FULL: all R steps exist.  FIN: some steps of the slab were captured into the final state
// (slot t - fin_first for t >= fin_first = L - S_out) and get that slot's gradient, read at `fin` (the lane's
// first channel of slot 0) where it is needed: at most S_out steps per sequence.
template <int DT, int W, bool MASK, bool ACT, bool FULL, bool FIN, int R, int E>
__device__ __forceinline__ void bwd_sweep(const BwdArgs &a, const float (*w)[W], const float *bias, const BVT *X,
                                          const BVT *H, const BVT *G, const float *mm, const float (*dzh)[E],
                                          float (*dzf)[E], float (*dw)[W], float *dbs, char *dxp, int64_t ds, int rows,
                                          bool active, const char *fin = nullptr, int64_t fin_first_row = 0)
{
    float xw[4][E];   // xm of rows r-3 .. r
#pragma unroll
    for (int k = 0; k < 4; ++k) unpack_half<DT>(X[R - 4 + k], xw[k]);
    // The residual's gradient is added before the mask multiply (masked residual) or after it (unmasked); with
    // nothing in between the two are the same sum.  Real branches (the empty asm keeps the compiler from turning
    // them into an add and a select per element and mode: 12 of 75 VALU instructions per row).
    const bool res_pre = a.res_mode == CANON_RESIDUAL_MASKED || (!MASK && !FIN && a.res_mode == CANON_RESIDUAL_UNMASKED);
    const bool res_post = a.res_mode == CANON_RESIDUAL_UNMASKED && !res_pre;
#pragma unroll
    for (int r = R - 1; r >= 0; --r) {
        float g[E], dz[E], o[E];
        unpack_half<DT>(G[r], g);
        if (r >= 3 || !ACT) {
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
        if (res_pre) {
            asm volatile("");
#pragma unroll
            for (int e = 0; e < E; ++e) o[e] += g[e];
        }
        if constexpr (FIN) {
            // fin_first_row: the slab row of the first captured step (may be negative)
            if (r >= fin_first_row && r < rows) {
#pragma unroll
                for (int e = 0; e < E; ++e)
                    o[e] += load1<DT>(fin, (int64_t)e * a.k_sc + ((int64_t)r - fin_first_row) * a.k_ss);
            }
        }
        if constexpr (MASK) {
            if (mm[3 + r] != 1.0f) {
#pragma unroll
                for (int e = 0; e < E; ++e) o[e] *= mm[3 + r];
            }
        }
        if (res_post) {
            asm volatile("");
#pragma unroll
            for (int e = 0; e < E; ++e) o[e] += g[e];
        }
        if ((FULL || r < rows) && active) BV::store<kBwdStream>(dxp + r * ds, pack_half<DT>(o));
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

// STATES: the call has an initial state or the gradient of a captured final state.  Its own instances: as
// run-time branches of one kernel the three pieces of code cost every call 30 registers and 100 scalar spills
// (B 8, C 3456, L 1024 without states: 38 -> 41 us).
template <int DT, int W, bool MASK, bool ACT, bool STATES>
__global__ __launch_bounds__(256) void canon_bwd_blc_kernel(const BwdArgs a)
{
    constexpr int BY = Elem<DT>::bytes;
    constexpr int E = kBwdVecBytes / BY;
    constexpr int R = kBwdSlab, NW = kBwdWaves;
    // With an activation: tailx / headdz, two barriers per tile (dz of a slab's head needs the previous
    // wave's tail first).  Without one dz IS dout, so the head is handed over as raw rows (headg) together
    // with the tail, one barrier per tile, both double-buffered (a fast wave publishes the next tile while
    // a slow one still reads this one).
    __shared__ BVT tailx[ACT ? 1 : 2][NW][3][64];            // last three xm rows of each wave's slab (storage bits)
    __shared__ float headdz[ACT ? NW : 1][3][ACT ? E : 1][64];  // dz of the first three steps of each wave's slab
    __shared__ BVT headg[2][ACT ? 1 : NW][3][64];            // ACT == false: the first three dout rows of each slab
    __shared__ float red[NW - 1][5 * E][64];      // dweight / dbias sums of waves 1..3
    // mask entries of steps t_chunk-3 .. t_chunk+chunk+2 as floats.  Staged once per block: inside the
    // time loop (after the first store to dx) the compiler can no longer use scalar loads for them, and
    // as vector loads in the tile's load group they cost 20 % of the kernel.
    __shared__ float smask[MASK ? kBwdMaxChunk + 6 : 1];

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
    fetch_taps<W, E>(a.weight, a.bias, a.w_sc, a.w_sk, a.w_dtype, a.w_vec != 0, c0, rawt);
    float w[E][W], bias[E];
    if constexpr (MASK) {
        for (uint32_t i = threadIdx.x; i < a.chunk + 6u; i += 64u * NW) {
            int64_t t = t_chunk - 3 + (int64_t)i;
            t = t < 0 ? 0 : (t > Lm1 ? Lm1 : t);
            smask[i] = load_mask(a.mask, (int64_t)b * a.m_sb + t * a.m_sl, a.mask_dtype);
        }
        __syncthreads();
    }

    // The tiles are walked from the last to the first, so the dz of the three steps after a tile
    // are the head of the tile done just before (still in headdz[0]).  For the chunk's last tile
    // the last wave computes them here, from six rows of x and three of dout, and leaves them
    // in that slot itself.
    float dzf[3][E];   // dzf[j] = dz[t + 1 + j] for the step t being processed
#pragma unroll
    for (int j = 0; j < 3; ++j)
#pragma unroll
        for (int e = 0; e < E; ++e) dzf[j][e] = 0.0f;
    if constexpr (!ACT) {
        // no activation: the three dz after the chunk are three rows of dout, kept by the last wave
        const int64_t te = t_chunk + (int64_t)a.chunk;
        BVT GE[3];
#pragma unroll
        for (int j = 0; j < 3; ++j) GE[j] = BV::zero();
        if (wv == NW - 1) {
#pragma unroll
            for (int j = 0; j < 3; ++j)
                if (te + j <= Lm1) GE[j] = BV::load<false>(gb + (te + j) * gs);
        }
        decode_taps<DT, W, E>(rawt, a.w_dtype, a.w_vec != 0, a.bias != nullptr, w, bias);
#pragma unroll
        for (int j = 0; j < 3; ++j) unpack_half<DT>(GE[j], dzf[j]);
    } else {
        const int64_t te = t_chunk + (int64_t)a.chunk;   // first step after the chunk (at least 32)
        BVT XE[6], GE[3];
        float me[6];
#pragma unroll
        for (int j = 0; j < 6; ++j) {
            XE[j] = BV::zero();
            me[j] = 1.0f;
        }
#pragma unroll
        for (int j = 0; j < 3; ++j) GE[j] = BV::zero();
        if (wv == NW - 1 && te <= Lm1) {
#pragma unroll
            for (int j = 0; j < 6; ++j) {
                const int64_t t = te - 3 + j;
                XE[j] = BV::load<false>(xb + (t < Lm1 ? t : Lm1) * xs);
            }
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                const int64_t t = te + j;
                GE[j] = BV::load<false>(gb + (t < Lm1 ? t : Lm1) * gs);
            }
            if constexpr (MASK) {
#pragma unroll
                for (int j = 0; j < 6; ++j) me[j] = smask[a.chunk + j];   // steps te-3 .. te+2
            }
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

    for (int it = ntiles - 1; it >= 0; --it) {
        const int64_t t0 = t_chunk + ((int64_t)it * NW + wv) * R;
        const int64_t left = (int64_t)a.L - t0;
        const int rows = left >= R ? R : (left > 0 ? (int)left : 0);   // wave uniform

        // ---- all loads of the tile.  Requesting the next tile's rows while this one is worked on was measured
        // three times (before, and after, this tile's rows are waited for; with two register sets taken in turn
        // and wait counts that leave the next tile's loads in flight): 3-5 % slower, 40-60 more registers.
        BVT X[R], G[R], H[3];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int64_t t = t0 + r < Lm1 ? t0 + r : Lm1;
            X[r] = BV::load<kBwdStream>(xb + t * xs);
            G[r] = BV::load<kBwdStream>(gb + t * gs);
        }
#pragma unroll
        for (int j = 0; j < 3; ++j) H[j] = BV::zero();
        if (wv == 0) {
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                const int64_t t = t0 - 3 + j;
                if (t >= 0) H[j] = BV::load<false>(xb + (t < Lm1 ? t : Lm1) * xs);
            }
        }
        float mm[R + 3];   // mask of steps t0-3 .. t0+R-1
#pragma unroll
        for (int j = 0; j < R + 3; ++j) mm[j] = 1.0f;
        if constexpr (MASK) {
            const uint32_t first = ((uint32_t)it * NW + wv) * R;   // index of step t0 - 3 in smask
#pragma unroll
            for (int j = 0; j < R + 3; ++j) mm[j] = smask[first + j];
        }

        // dz of the three steps after the slab; the last wave's are the previous iteration's head of wave 0
        const int pb = it & 1;   // ACT == false: LDS buffer of this tile
        if constexpr (ACT) {
            if (wv == NW - 1) {
#pragma unroll
                for (int j = 0; j < 3; ++j)
#pragma unroll
                    for (int e = 0; e < E; ++e) dzf[j][e] = headdz[0][j][e][lane];
            }
        } else {
            if (wv == NW - 1 && it != ntiles - 1) {   // (the chunk's last tile: the rows loaded before the loop)
#pragma unroll
                for (int j = 0; j < 3; ++j) unpack_half<DT>(headg[pb ^ 1][0][j][lane], dzf[j]);
            }
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
        if (STATES && a.init && t0 == 0 && wv == 0) {
            // rows before t = 0: entries of the initial state, not masked
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                const int s_ = a.S_in - 3 + j;
                if (s_ < 0) continue;
                float f[E];
#pragma unroll
                for (int e = 0; e < E; ++e)
                    f[e] = load1<DT>(a.init, (int64_t)b * a.i_sb + (int64_t)(c0 + e) * a.i_sc + (int64_t)s_ * a.i_ss);
                H[j] = pack_half<DT>(f);
            }
        }
        if constexpr (!ACT) {
            // tail of x and head of dout (zero past the end of the sequence) in one exchange
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                tailx[pb][wv][j][lane] = X[R - 3 + j];
                headg[pb][wv][j][lane] = j < rows ? G[j] : BV::zero();
            }
            __syncthreads();
            if (wv > 0) {
#pragma unroll
                for (int j = 0; j < 3; ++j) H[j] = tailx[pb][wv - 1][j][lane];
            }
            if (wv < NW - 1) {
#pragma unroll
                for (int j = 0; j < 3; ++j) unpack_half<DT>(headg[pb][wv + 1][j][lane], dzf[j]);
            }
        }
        float dzh[3][E];
#pragma unroll
        for (int j = 0; j < 3; ++j)
#pragma unroll
            for (int e = 0; e < E; ++e) dzh[j][e] = 0.0f;   // (unused without an activation)
        if constexpr (ACT) {
#pragma unroll
            for (int j = 0; j < 3; ++j) tailx[0][wv][j][lane] = X[R - 3 + j];
            __syncthreads();
            if (wv > 0) {
#pragma unroll
                for (int j = 0; j < 3; ++j) H[j] = tailx[0][wv - 1][j][lane];
            }

            // ---- dz of the slab's first three steps, handed to the previous wave ---------
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
        }

        // ---- sweep the slab from its last step to its first --------------------------
        const int64_t fin_first = (int64_t)a.L - a.S_out;   // first captured step (S_out is 0 without dfinal_state)
        if (STATES && a.dfin && t0 + rows > fin_first) {
            // slot 0 of the final state's gradient holds step fin_first
            const char *fin = a.dfin + ((int64_t)b * a.k_sb + (int64_t)c0 * a.k_sc) * BY;
            bwd_sweep<DT, W, MASK, ACT, false, true, R, E>(a, w, bias, X, H, G, mm, dzh, dzf, dw, dbs, db_ + t0 * ds, ds, rows,
                                                           active, fin, fin_first - t0);
        } else if (rows == R)
            bwd_sweep<DT, W, MASK, ACT, true, false, R, E>(a, w, bias, X, H, G, mm, dzh, dzf, dw, dbs, db_ + t0 * ds, ds, rows, active);
        else
            bwd_sweep<DT, W, MASK, ACT, false, false, R, E>(a, w, bias, X, H, G, mm, dzh, dzf, dw, dbs, db_ + t0 * ds, ds, rows, active);
    }

    if (STATES && a.dinit && ch == 0 && wv == 0 && active) {
        // here dzf[i] = dz[i] (zero past the end of the row).  Entry s is the input at t = s - S_in = -d:
        // its gradient is sum_i w[W-1-d-i] * dz[i] over the taps that exist
        for (int s_ = 0; s_ < a.S_in; ++s_) {
            const int d = a.S_in - s_;
            // a final state longer than the row also captured this entry (input at t = -d) in slot S_out - L - d
            const int64_t slot = (int64_t)a.S_out - (int64_t)a.L - d;
#pragma unroll
            for (int e = 0; e < E; ++e) {
                float acc = 0.0f;
#pragma unroll
                for (int i = 0; i < 3; ++i) {
                    const int k = W - 1 - d - i;
                    if (k >= 0) acc = fmaf(w[e][k < 0 ? 0 : k], dzf[i][e], acc);
                }
                if (a.dfin && slot >= 0)
                    acc += load1<DT>(a.dfin, (int64_t)b * a.k_sb + (int64_t)(c0 + e) * a.k_sc + slot * a.k_ss);
                store1<DT>(a.dinit, (int64_t)b * a.j_sb + (int64_t)(c0 + e) * a.j_sc + (int64_t)s_ * a.j_ss, acc);
            }
        }
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

// The scalars in front of the argument block are what a wave needs to request its rows of x and dout; they arrive in
// registers with the wave (kernel-argument preload), so the loads are issued without a read of the argument block in
// front of them, as in the forward kernel.  g_sb / g_sc: the strides of dout when they differ from x's, else a copy
// of x's; `divC_s`: s1 | s2 << 1 of the division by C.
template <int DT, int W, int U, bool MASK>
__global__ __launch_bounds__(256) void canon_bwd_bcl_kernel(const char *x_base, const char *g_base, uint32_t x_sb32,
                                                            uint32_t x_sc32, uint32_t g_sb32, uint32_t g_sc32,
                                                            uint32_t nthreads, uint32_t nchunk, uint32_t C, uint32_t divC_m,
                                                            uint32_t divC_s, uint32_t nvec, const BwdArgs a)
{
    constexpr int E = Elem<DT>::per_vec;
    constexpr int BY = Elem<DT>::bytes;
    const int lane = threadIdx.x & 63;
    const uint32_t task = __builtin_amdgcn_readfirstlane(blockIdx.x * 4u + (threadIdx.x >> 6));
    if (task >= nthreads) return;            // nthreads = wave tasks in this kernel
    uint32_t row = task, seg = 0;
    if (nchunk > 1) {                        // nchunk = segments per row
        row = fdiv(task, a.div_nchunk);
        seg = task - row * nchunk;
    }
    const uint32_t b = fdiv(row, FastDiv{C, divC_m, divC_s & 1u, divC_s >> 1});
    const uint32_t c = row - b * C;

    // (strides in vectors of E elements: the planner takes this kernel only for rows that start on 16-byte boundaries)
    const char *xrow = x_base + ((int64_t)b * x_sb32 + (int64_t)c * x_sc32) * 16;
    const char *grow = g_base + ((int64_t)b * g_sb32 + (int64_t)c * g_sc32) * 16;
    char *drow = a.dx + ((int64_t)b * a.d_sb + (int64_t)c * a.d_sc) * BY;
    const uint32_t v0 = seg * (64u * U) + lane;

    uint4 X[U], G[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t v = v0 + u * 64u;
        const uint32_t vc = v < nvec ? v : nvec - 1u;
        X[u] = load_vec<kBwdStream>(xrow + (int64_t)vc * 16);
        G[u] = load_vec<kBwdStream>(grow + (int64_t)vc * 16);
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
        if (v < nvec) store_vec<kBwdStream>(drow + (int64_t)v * 16, pack_vec<DT>(o));
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
    if (i < ncols) {
        uint32_t s = slice;
        for (; s + 24u < nsets; s += 32u) {   // four loads in flight, added in set order
            const float v0 = partial[(int64_t)s * ncols + i], v1 = partial[(int64_t)(s + 8u) * ncols + i];
            const float v2 = partial[(int64_t)(s + 16u) * ncols + i], v3 = partial[(int64_t)(s + 24u) * ncols + i];
            acc += (double)v0;
            acc += (double)v1;
            acc += (double)v2;
            acc += (double)v3;
        }
        for (; s < nsets; s += 8u) acc += (double)partial[(int64_t)s * ncols + i];
    }
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
// backward of one decode step (shift-register state).  A thread owns one
// channel and walks the batch entries of its group in order, so a wave reads
// dense stretches of x / dout / the state and the partial sums of dweight /
// dbias it leaves per group are formed in a fixed order; canon_bwd_reduce_kernel
// then sums the groups.  z is recomputed from the saved state and the token.
// ---------------------------------------------------------------------------
// Taps, window and sums are kept right-aligned in arrays of four (tap k of a width-W filter at index
// 4-W+k, the token's tap always at 3, window entry i = state slot S-3+i), so every register array is
// indexed by compile-time constants whatever W is.
template <int DT>
__device__ __forceinline__ void load_taps_right(const UpdBwdArgs &a, uint32_t c, float *wr, float &bv)
{
    const int lead = 4 - a.W;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        wr[i] = i >= lead ? round_through<DT>(load_w(a.weight, (int64_t)c * a.w_sc + (i - lead) * a.w_sk, a.w_dtype)) : 0.0f;
    bv = a.bias ? round_through<DT>(load_w(a.bias, c, a.w_dtype)) : 0.0f;
}

// one (batch entry, channel): wn[i] = state slot S-3+i (0 where no tap reads it), qr[i] = gradient of the updated
// state at slot S-4+i (qr[3]: the token's own slot).  Returns dz; dx in dxv; adds to the sums.
__device__ __forceinline__ float update_bwd_point(const UpdBwdArgs &a, const float *wr, float bv, const float *wn,
                                                  const float *qr, float xr, float xt, float go, float m, float *dwr,
                                                  float &db, float &dxv)
{
    float dz = go;
    if (a.act) {
        float z = bv;
#pragma unroll
        for (int i = 0; i < 3; ++i) z = fmaf(wr[i], wn[i], z);
        z = fmaf(wr[3], xt, z);
        dz = go * silu_grad(z);
    }
#pragma unroll
    for (int i = 0; i < 3; ++i) dwr[i] = fmaf(dz, wn[i], dwr[i]);
    dwr[3] = fmaf(dz, xt, dwr[3]);
    db += dz;
    float dxt = wr[3] * dz;
    if (a.res_mode == CANON_RESIDUAL_MASKED) dxt += go;
    dxt += qr[3];
    dxv = a.tmask ? dxt * m : dxt;
    if (a.res_mode == CANON_RESIDUAL_UNMASKED) dxv += go;
    return dz;
}

__device__ __forceinline__ void store_partial_right(const UpdBwdArgs &a, float *pp, const float *dwr, float db)
{
    const int lead = 4 - a.W;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        float v = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (i - lead == k) v = dwr[i];
        pp[k] = v;
    }
    pp[4] = db;
}

// Ring-buffer mode (seqlens): the forward wrote the token to slot p = seqlens[b] mod S and read the W-1 slots before
// it cyclically, every other slot stayed where it was.  That is the shift register seen through a rotation: entry j
// of the state before the step lives in slot (p + j) mod S, entry i of the state after it in slot (p + 1 + i) mod S,
// so the code below is written in shift-register entries and maps them to slots where it touches memory.
// State-pool mode (indices): batch entry b uses row indices[b] of conv_state / dstate_out / dstate; an entry whose
// index lies outside the pool was skipped by the forward (its output is a constant zero row): dx = 0, nothing else.
// Only the rows the entries name are written: the caller fills dstate with dstate_out (or zeros) beforehand, so that
// the rows no entry used pass their gradient through.
template <int DT>
__global__ __launch_bounds__(256) void canon_update_bwd_kernel(const UpdBwdArgs a)
{
    constexpr int NB = 4;                   // batch entries whose loads are requested together
    const uint32_t c = blockIdx.x * 256u + threadIdx.x;
    if (c >= a.C) return;
    const uint32_t g = blockIdx.y;
    const int S = a.S;
    const int lead = 4 - a.W;               // window entries / taps below this index do not exist
    float wr[4], bv;
    load_taps_right<DT>(a, c, wr, bv);
    float dwr[4] = {0, 0, 0, 0}, db = 0.0f;
    const uint32_t b_begin = g * a.group;
    const uint32_t b_stop = b_begin + a.group < a.B ? b_begin + a.group : a.B;
    for (uint32_t b0 = b_begin; b0 < b_stop; b0 += NB) {
        // every load of the NB entries first (nothing is stored in between, so they are in flight together)
        float xr[NB], go[NB], m[NB], wn[NB][3], qr[NB][4];
        int64_t row[NB];                    // row of the state tensors, -1: entry skipped
        int pos[NB];                        // ring: slot of the token, else -1
#pragma unroll
        for (int n = 0; n < NB; ++n) {
            const uint32_t b = b0 + n < b_stop ? b0 + n : b_stop - 1u;
            row[n] = b;
            if (a.indices) {
                const int32_t i = a.indices[b];
                row[n] = (i < 0 || (a.state_rows > 0 && (uint32_t)i >= a.state_rows)) ? -1 : i;
            }
            pos[n] = -1;
            if (a.seqlens) {
                pos[n] = a.seqlens[b] % S;
                if (pos[n] < 0) pos[n] += S;
            }
            const bool live = row[n] >= 0;
            // slots of entry j of the state before the step and of entry e of the state after it
            auto slot = [&](int j) { return pos[n] < 0 ? j : (pos[n] + j) % S; };
            auto slot_after = [&](int e) { return pos[n] < 0 ? e : (pos[n] + 1 + e) % S; };
            xr[n] = load1<DT>(a.x, (int64_t)b * a.x_sb + (int64_t)c * a.x_sc);
            go[n] = live ? load1<DT>(a.dy, (int64_t)b * a.g_sb + (int64_t)c * a.g_sc) : 0.0f;
            m[n] = a.tmask ? load_mask(a.tmask, (int64_t)b * a.m_sb, a.mask_dtype) : 1.0f;
            const int64_t so = row[n] * a.s_sb + (int64_t)c * a.s_sc;
            const int64_t qo = row[n] * a.q_sb + (int64_t)c * a.q_sc;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (i < 3) wn[n][i] = (live && i >= lead) ? load1<DT>(a.state, so + (int64_t)slot(S - 3 + i) * a.s_ss) : 0.0f;
                qr[n][i] = (live && a.dso && i >= lead && S - 4 + i >= 0) ? load1<DT>(a.dso, qo + (int64_t)slot_after(S - 4 + i) * a.q_ss) : 0.0f;
            }
        }
#pragma unroll
        for (int n = 0; n < NB; ++n) {
            const uint32_t b = b0 + n;
            if (b >= b_stop) break;
            if (row[n] < 0) {
                store1<DT>(a.dx, (int64_t)b * a.d_sb + (int64_t)c * a.d_sc, 0.0f);
                continue;
            }
            auto slot = [&](int j) { return pos[n] < 0 ? j : (pos[n] + j) % S; };
            auto slot_after = [&](int e) { return pos[n] < 0 ? e : (pos[n] + 1 + e) % S; };
            const float xt = a.tmask ? mul_round<DT>(xr[n], m[n]) : xr[n];
            float dxv;
            const float dz = update_bwd_point(a, wr, bv, wn[n], qr[n], xr[n], xt, go[n], m[n], dwr, db, dxv);
            store1<DT>(a.dx, (int64_t)b * a.d_sb + (int64_t)c * a.d_sc, dxv);
            if (a.ds) {
                const int64_t ro = row[n] * a.r_sb + (int64_t)c * a.r_sc;
                const int64_t qo = row[n] * a.q_sb + (int64_t)c * a.q_sc;
                // entries no tap reads: the gradient of the updated state one entry earlier (the same slot of a ring)
                for (int j = 0; j < S - 3 + lead; ++j)
                    store1<DT>(a.ds, ro + (int64_t)slot(j) * a.r_ss,
                               (a.dso && j >= 1) ? load1<DT>(a.dso, qo + (int64_t)slot_after(j - 1) * a.q_ss) : 0.0f);
#pragma unroll
                for (int i = 0; i < 3; ++i)
                    if (i >= lead) store1<DT>(a.ds, ro + (int64_t)slot(S - 3 + i) * a.r_ss, fmaf(wr[i], dz, qr[n][i]));
            }
        }
    }
    if (a.partial) store_partial_right(a, a.partial + ((int64_t)g * a.C + c) * 5, dwr, db);
}

// The same for a contiguous [B, C, S] state (and state gradients), S = 3 or 4, channel-contiguous token / dout /
// dx: a lane owns E adjacent channels (two of a 16-bit type, one fp32) whose state rows are ONE run of 12 or
// 16 bytes, as in the forward kernel, so every access of a wave is a dense stretch read or written whole.
// The four waves of a block share a 64-lane channel tile and take every fourth batch entry of the block's
// group; their sums are added in wave order through LDS, so a group is 4 x as many entries (a quarter of the
// partial sets) for the same work per wave.
template <int DT, int S>
__global__ __launch_bounds__(256) void canon_update_bwd_vec_kernel(const UpdBwdArgs a)
{
    constexpr int NB = 4;                   // batch entries whose loads are requested together
    constexpr int BY = Elem<DT>::bytes;
    constexpr int E = upd_lane_channels(BY, S);
    constexpr int ND = E * S * BY / 4;      // words of state per lane and batch entry
    static_assert(E * BY == 4 && (S == 3 || S == 4), "one word of token / dout / dx per lane");
    __shared__ float sums[3][64][E * 5 + 1];   // waves 1..3 hand their sums to wave 0 (+1: no bank conflicts)
    const uint32_t lane = threadIdx.x & 63u, wv = threadIdx.x >> 6;
    const uint32_t cv = blockIdx.x * 64u + lane;
    const uint32_t c0 = cv * E;
    const bool live = c0 < a.C;
    const uint32_t g = blockIdx.y;
    const int lead = 4 - a.W;
    float wr[E][4], bv[E], dwr[E][4], db[E];
#pragma unroll
    for (int e = 0; e < E; ++e) {
        if (live) load_taps_right<DT>(a, c0 + e, wr[e], bv[e]);
        db[e] = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) dwr[e][i] = 0.0f;
    }
    const uint32_t b_begin = g * a.group;
    const uint32_t b_stop = b_begin + a.group < a.B ? b_begin + a.group : a.B;
    // this wave's entries: b_begin + wv, + 4, + 8, ...
    for (uint32_t b0 = b_begin + wv; live && b0 < b_stop; b0 += 4u * NB) {
        uint32_t X[NB], G[NB], ST[NB][ND], Q[NB][ND];
        float m[NB];
#pragma unroll
        for (int n = 0; n < NB; ++n) {
            const uint32_t bn = b0 + 4u * n;
            const uint32_t b = bn < b_stop ? bn : b0;
            X[n] = *(const uint32_t *)(a.x + ((int64_t)b * a.x_sb + c0) * BY);
            G[n] = *(const uint32_t *)(a.dy + ((int64_t)b * a.g_sb + c0) * BY);
            load_words<ND>(a.state + ((int64_t)b * a.s_sb + (int64_t)c0 * S) * BY, ST[n]);
            if (a.dso) {
                load_words<ND>(a.dso + ((int64_t)b * a.q_sb + (int64_t)c0 * S) * BY, Q[n]);
            } else {
#pragma unroll
                for (int i = 0; i < ND; ++i) Q[n][i] = 0u;
            }
            m[n] = a.tmask ? load_mask(a.tmask, (int64_t)b * a.m_sb, a.mask_dtype) : 1.0f;
        }
#pragma unroll
        for (int n = 0; n < NB; ++n) {
            const uint32_t b = b0 + 4u * n;
            if (b >= b_stop) break;
            uint32_t ox = 0u, DS[ND];
#pragma unroll
            for (int i = 0; i < ND; ++i) DS[i] = 0u;
#pragma unroll
            for (int e = 0; e < E; ++e) {
                const float xr = Packed<DT>::as_float(Packed<DT>::get(&X[n], e));
                const float go = Packed<DT>::as_float(Packed<DT>::get(&G[n], e));
                const float xt = a.tmask ? mul_round<DT>(xr, m[n]) : xr;
                float wn[3], qr[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (i < 3) wn[i] = i >= lead ? Packed<DT>::as_float(Packed<DT>::get(ST[n], e * S + S - 3 + i)) : 0.0f;
                    qr[i] = (i >= lead && S - 4 + i >= 0) ? Packed<DT>::as_float(Packed<DT>::get(Q[n], e * S + (S - 4 + i >= 0 ? S - 4 + i : 0))) : 0.0f;
                }
                float dxv;
                const float dz = update_bwd_point(a, wr[e], bv[e], wn, qr, xr, xt, go, m[n], dwr[e], db[e], dxv);
                Packed<DT>::put(&ox, e, Packed<DT>::raw_of(dxv));
                // slots no tap reads: the gradient of the updated state shifted by one (raw bits); the others
                // add their tap's share
#pragma unroll
                for (int j = 0; j < S; ++j) {
                    const int i = j - (S - 3);
                    uint32_t raw = j >= 1 ? Packed<DT>::get(Q[n], e * S + (j >= 1 ? j - 1 : 0)) : 0u;
                    if (i >= 0 && i >= lead) raw = Packed<DT>::raw_of(fmaf(wr[e][i >= 0 ? i : 0], dz, qr[i >= 0 ? i : 0]));
                    Packed<DT>::put(DS, e * S + j, raw);
                }
            }
            *(uint32_t *)(a.dx + ((int64_t)b * a.d_sb + c0) * BY) = ox;
            if (a.ds) store_words<ND>(a.ds + ((int64_t)b * a.r_sb + (int64_t)c0 * S) * BY, DS);
        }
    }
    if (!a.partial) return;                 // uniform over the block
    if (wv != 0) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
#pragma unroll
            for (int i = 0; i < 4; ++i) sums[wv - 1][lane][e * 5 + i] = dwr[e][i];
            sums[wv - 1][lane][e * 5 + 4] = db[e];
        }
    }
    __syncthreads();
    if (wv != 0 || !live) return;
#pragma unroll
    for (int k = 0; k < 3; ++k) {           // wave order: a fixed order of additions
#pragma unroll
        for (int e = 0; e < E; ++e) {
#pragma unroll
            for (int i = 0; i < 4; ++i) dwr[e][i] += sums[k][lane][e * 5 + i];
            db[e] += sums[k][lane][e * 5 + 4];
        }
    }
#pragma unroll
    for (int e = 0; e < E; ++e) store_partial_right(a, a.partial + ((int64_t)g * a.C + c0 + e) * 5, dwr[e], db[e]);
}

// ---------------------------------------------------------------------------
// launch
// ---------------------------------------------------------------------------
namespace {

template <int DT, int W, bool MASK> void launch_bwd_m(const BwdPlan &pl, hipStream_t s)
{
    const dim3 g(pl.grid), b(256);
    if (pl.kind == BWD_BCL_VEC) {
        const BwdArgs &A = pl.args;
        constexpr int64_t EV = Elem<DT>::per_vec;
        switch (pl.U) {
#define CANON_BWD_BCL_LAUNCH(UU)                                                                                         \
    hipLaunchKernelGGL((canon_bwd_bcl_kernel<DT, W, UU, MASK>), g, b, 0, s, A.x, A.dy, (uint32_t)(A.x_sb / EV),         \
                       (uint32_t)(A.x_sc / EV), (uint32_t)(A.g_sb / EV), (uint32_t)(A.g_sc / EV), A.nthreads, A.nchunk,  \
                       A.C, A.div_nvec.m, A.div_nvec.s1 | A.div_nvec.s2 << 1, A.L / (uint32_t)EV, A)
        case 4: CANON_BWD_BCL_LAUNCH(4); break;
        case 2: CANON_BWD_BCL_LAUNCH(2); break;
        default: CANON_BWD_BCL_LAUNCH(1); break;
#undef CANON_BWD_BCL_LAUNCH
        }
    } else if (pl.kind == BWD_BLC_VEC)
    {
        const bool states = pl.args.init != nullptr || pl.args.dfin != nullptr;
        if (pl.args.act) {
            if (states) hipLaunchKernelGGL((canon_bwd_blc_kernel<DT, W, MASK, true, true>), g, b, 0, s, pl.args);
            else hipLaunchKernelGGL((canon_bwd_blc_kernel<DT, W, MASK, true, false>), g, b, 0, s, pl.args);
        } else {
            if (states) hipLaunchKernelGGL((canon_bwd_blc_kernel<DT, W, MASK, false, true>), g, b, 0, s, pl.args);
            else hipLaunchKernelGGL((canon_bwd_blc_kernel<DT, W, MASK, false, false>), g, b, 0, s, pl.args);
        }
    }
    else if (pl.args.seq)
        hipLaunchKernelGGL((canon_bwd_walk_kernel<DT, W, MASK, kBwdRows, true>), g, b, 0, s, pl.args);
    else
        hipLaunchKernelGGL((canon_bwd_walk_kernel<DT, W, MASK, kBwdRows, false>), g, b, 0, s, pl.args);
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

}  // namespace

void launch_bwd(const BwdPlan &pl, int x_dtype, hipStream_t s)
{
    switch (x_dtype) {
    case CANON_DTYPE_F32: launch_bwd<CANON_DTYPE_F32>(pl, s); break;
    case CANON_DTYPE_BF16: launch_bwd<CANON_DTYPE_BF16>(pl, s); break;
    default: launch_bwd<CANON_DTYPE_F16>(pl, s); break;
    }
    hipLaunchKernelGGL(canon_bwd_reduce_kernel, dim3((pl.args.C * 5u + 31u) / 32u), dim3(256), 0, s,
                       pl.args.partial, pl.args.dweight, pl.args.dbias, pl.args.C, pl.args.nsets, pl.args.W);
}

void launch_update_bwd(const UpdBwdPlan &pl, int x_dtype, hipStream_t s)
{
    const dim3 g(pl.grid_c, pl.args.ngroups), b(256);   // vec: 64 lanes of channels per block, else 256 channels
    if (pl.vec) {
        const bool s3 = pl.args.S == 3;
        switch (x_dtype) {
        case CANON_DTYPE_F32:
            if (s3) hipLaunchKernelGGL((canon_update_bwd_vec_kernel<CANON_DTYPE_F32, 3>), g, b, 0, s, pl.args);
            else hipLaunchKernelGGL((canon_update_bwd_vec_kernel<CANON_DTYPE_F32, 4>), g, b, 0, s, pl.args);
            break;
        case CANON_DTYPE_BF16:
            if (s3) hipLaunchKernelGGL((canon_update_bwd_vec_kernel<CANON_DTYPE_BF16, 3>), g, b, 0, s, pl.args);
            else hipLaunchKernelGGL((canon_update_bwd_vec_kernel<CANON_DTYPE_BF16, 4>), g, b, 0, s, pl.args);
            break;
        default:
            if (s3) hipLaunchKernelGGL((canon_update_bwd_vec_kernel<CANON_DTYPE_F16, 3>), g, b, 0, s, pl.args);
            else hipLaunchKernelGGL((canon_update_bwd_vec_kernel<CANON_DTYPE_F16, 4>), g, b, 0, s, pl.args);
            break;
        }
    } else {
        switch (x_dtype) {
        case CANON_DTYPE_F32: hipLaunchKernelGGL((canon_update_bwd_kernel<CANON_DTYPE_F32>), g, b, 0, s, pl.args); break;
        case CANON_DTYPE_BF16: hipLaunchKernelGGL((canon_update_bwd_kernel<CANON_DTYPE_BF16>), g, b, 0, s, pl.args); break;
        default: hipLaunchKernelGGL((canon_update_bwd_kernel<CANON_DTYPE_F16>), g, b, 0, s, pl.args); break;
        }
    }
    if (pl.args.partial)
        hipLaunchKernelGGL(canon_bwd_reduce_kernel, dim3((pl.args.C * 5u + 31u) / 32u), dim3(256), 0, s, pl.args.partial,
                           pl.args.dweight, pl.args.dbias, pl.args.C, pl.args.ngroups, pl.args.W);
}

// Asking for a kernel's attributes makes the runtime load this file's code object onto the current device.
hipError_t preload_bwd()
{
    hipFuncAttributes attr;
    return hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(&canon_zero_kernel));
}

void launch_zero(float *p, uint32_t n, hipStream_t s)
{
    if (n) hipLaunchKernelGGL(canon_zero_kernel, dim3((n + 255) / 256), dim3(256), 0, s, p, n);
}

}  // namespace canon
