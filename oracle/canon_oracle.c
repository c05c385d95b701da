/*
 * CPU oracle for the Canon causal depthwise conv1d (prefill + decode update).
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP kernels are
 * compared against; nothing in the shipped library links or calls it.
 *
 * What it restates (reference = JohanLi233/Viby-Model):
 *   - prefill math      model/model.py:590-675 (eager CanonLayer: mask multiply,
 *                       F.pad(W-1,0) + F.conv1d(groups=C), optional F.silu,
 *                       residual), causal-conv1d-mps/test.py:83-107 (fp32
 *                       oracle of the submodule's tests), tap order and single
 *                       rounding of causal_conv1d_mps/causal_conv1d.metal:229-272
 *                       and :530-580
 *   - state capture     model/model.py:470-489 and :623-661
 *   - decode update     model/model.py:372-398 (_pytorch_step: shift left by
 *                       one, append, dot with the taps) and the call contract
 *                       at model/model.py:305-311
 *   - bf16 rounding     causal_conv1d.metal:100-127 (RNE, NaN -> quiet NaN)
 *
 * Arithmetic contract (measured against torch CPU, which evaluates the fp32
 * depthwise conv as exactly this chain):
 *     acc = bias[c]                       (0.0f when there is no bias)
 *     for k = 0 .. W-1:  acc = fmaf(w[c][k], xm[t-(W-1)+k], acc)
 * where xm is the (optionally masked) input, zero for t < 0 unless an
 * initial state supplies the history.  Taps and bias are first rounded to
 * the storage type of x, as the reference wrappers cast them
 * (causal_conv1d_mps/__init__.py:136-140).
 *
 * round_mode 0 ("fused"):  SiLU and the residual add stay in fp32 and the
 *                          result is rounded to the storage type once.
 * round_mode 1 ("eager"):  the result is rounded to the storage type after
 *                          the conv, after SiLU and after the residual add,
 *                          the rounding points of the eager module.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

enum { CANON_F32 = 0, CANON_BF16 = 1, CANON_F16 = 2 };

static float bits_to_float(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t float_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static float bf16_to_float(uint16_t h) { return bits_to_float((uint32_t)h << 16); }

static uint16_t float_to_bf16(float f)
{
    uint32_t u = float_to_bits(f);
    if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x007FFFFFu) != 0)
        return (uint16_t)(((u >> 16) & 0x8000u) | 0x7FC0u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static float f16_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return bits_to_float(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-8f;
        return sign ? -v : v;
    }
    if (exp == 31) return bits_to_float(sign | 0x7F800000u | (man << 13));
    return bits_to_float(sign | ((exp + 112u) << 23) | (man << 13));
}

static uint16_t float_to_f16(float f)
{
    uint32_t u = float_to_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a >= 0x7F800000u) /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | (a > 0x7F800000u ? (0x0200u | ((a >> 13) & 0x3FFu)) : 0));
    if (a >= 0x477FF000u) /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7C00u);
    if (a < 0x33000001u) /* <= 2^-25 rounds to zero */
        return sign;
    int32_t e = (int32_t)(a >> 23) - 127;
    uint32_t m = (a & 0x007FFFFFu) | 0x00800000u;
    if (e < -14) {
        /* subnormal half: shift so that the unit is 2^-24 */
        int shift = 13 + (-14 - e);
        uint32_t q = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    uint32_t q = ((uint32_t)(e + 15) << 10) | ((m >> 13) & 0x3FFu);
    uint32_t rem = m & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++;
    return (uint16_t)(sign | q);
}

static float load_elem(const void *p, int64_t i, int dtype)
{
    switch (dtype) {
    case CANON_F32: return ((const float *)p)[i];
    case CANON_BF16: return bf16_to_float(((const uint16_t *)p)[i]);
    default: return f16_to_float(((const uint16_t *)p)[i]);
    }
}

static void store_elem(void *p, int64_t i, int dtype, float v)
{
    switch (dtype) {
    case CANON_F32: ((float *)p)[i] = v; break;
    case CANON_BF16: ((uint16_t *)p)[i] = float_to_bf16(v); break;
    default: ((uint16_t *)p)[i] = float_to_f16(v); break;
    }
}

/* value -> storage type -> value */
static float round_to(float v, int dtype)
{
    switch (dtype) {
    case CANON_F32: return v;
    case CANON_BF16: return bf16_to_float(float_to_bf16(v));
    default: return f16_to_float(float_to_f16(v));
    }
}

static float silu(float v) { return v / (1.0f + expf(-v)); }

/* Exposed so the tests can pin the conversions against torch. */
uint16_t canon_oracle_float_to_bf16(float f) { return float_to_bf16(f); }
uint16_t canon_oracle_float_to_f16(float f) { return float_to_f16(f); }
float canon_oracle_bf16_to_float(uint16_t h) { return bf16_to_float(h); }
float canon_oracle_f16_to_float(uint16_t h) { return f16_to_float(h); }

/*
 * Prefill.  All tensors contiguous:
 *   x, out        [B, C, L]   storage type `dtype`
 *   weight        [C, W]      storage type `w_dtype`;  bias [C] or NULL
 *   mask          [B, L] float32 or NULL  (xm = round(x * mask))
 *   init_state    [B, C, S_in]  or NULL   (history before t = 0: its last W-1)
 *   final_state   [B, C, S_out] or NULL   (last S_out of init_state ++ xm,
 *                                           zero filled on the left)
 *   residual_mode 0 none, 1 add the masked input, 2 add the unmasked input
 * Returns 0, or -1 for an argument the restatement does not cover.
 */
int canon_oracle_fwd(const void *x, const void *weight, const void *bias, const float *mask,
                     const void *init_state, void *out, void *final_state,
                     int64_t B, int64_t C, int64_t L, int W, int S_in, int S_out,
                     int dtype, int w_dtype, int use_silu, int residual_mode, int round_mode)
{
    if (W < 1 || W > 8 || B < 0 || C < 0 || L < 0) return -1;
    if (init_state && S_in < W - 1) return -1;
    for (int64_t b = 0; b < B; ++b) {
        for (int64_t c = 0; c < C; ++c) {
            float w[8];
            for (int k = 0; k < W; ++k) w[k] = round_to(load_elem(weight, c * W + k, w_dtype), dtype);
            const float bv = bias ? round_to(load_elem(bias, c, w_dtype), dtype) : 0.0f;
            const int64_t row = (b * C + c) * L;
            /* window[k] holds xm[t-(W-1)+k] */
            float window[8];
            for (int k = 0; k < W - 1; ++k)
                window[k + 1] = init_state
                    ? load_elem(init_state, (b * C + c) * S_in + (S_in - (W - 1) + k), dtype)
                    : 0.0f;
            for (int64_t t = 0; t < L; ++t) {
                const float xr = load_elem(x, row + t, dtype);
                float xm = xr;
                if (mask) xm = round_to(xr * mask[b * L + t], dtype);
                for (int k = 0; k < W - 1; ++k) window[k] = window[k + 1];
                window[W - 1] = xm;
                float acc = bv;
                for (int k = 0; k < W; ++k) acc = fmaf(w[k], window[k], acc);
                if (round_mode) acc = round_to(acc, dtype);
                if (use_silu) {
                    acc = silu(acc);
                    if (round_mode) acc = round_to(acc, dtype);
                }
                if (residual_mode) acc += (residual_mode == 1) ? xm : xr;
                store_elem(out, row + t, dtype, acc);
            }
            if (final_state) {
                for (int j = 0; j < S_out; ++j) {
                    const int64_t src = L - S_out + j; /* time index into x */
                    float v = 0.0f;
                    if (src >= 0) {
                        v = load_elem(x, row + src, dtype);
                        if (mask) v = round_to(v * mask[b * L + src], dtype);
                    } else if (init_state && S_in + src >= 0) {
                        v = load_elem(init_state, (b * C + c) * S_in + (S_in + src), dtype);
                    }
                    store_elem(final_state, (b * C + c) * S_out + j, dtype, v);
                }
            }
        }
    }
    return 0;
}

/*
 * Prefill over packed variable-length sequences: seq_idx [B, L] (int32) names
 * the sequence every position belongs to, and an input only contributes to
 * outputs of its own sequence (the `seq_idx` slot of causal_conv1d_fn; the
 * reference passes None, model/model.py:465, and its MPS backend rejects it,
 * causal_conv1d_mps/autograd.py:64-65, so this follows the published
 * behaviour of the upstream package: a tap whose input position carries
 * another index adds weight * 0).  No initial / final state in this mode.
 * PARITY UNPINNED against upstream (absent from the reference tree); pinned by
 * the defining property that a packed row equals its sequences run one by one.
 */
int canon_oracle_fwd_seq(const void *x, const void *weight, const void *bias, const float *mask,
                         const int32_t *seq_idx, void *out, int64_t B, int64_t C, int64_t L, int W,
                         int dtype, int w_dtype, int use_silu, int residual_mode)
{
    if (W < 1 || W > 8 || B < 0 || C < 0 || L < 0 || !seq_idx) return -1;
    for (int64_t b = 0; b < B; ++b) {
        for (int64_t c = 0; c < C; ++c) {
            float w[8];
            for (int k = 0; k < W; ++k) w[k] = round_to(load_elem(weight, c * W + k, w_dtype), dtype);
            const float bv = bias ? round_to(load_elem(bias, c, w_dtype), dtype) : 0.0f;
            const int64_t row = (b * C + c) * L;
            for (int64_t t = 0; t < L; ++t) {
                const float xr = load_elem(x, row + t, dtype);
                const float xm_t = mask ? round_to(xr * mask[b * L + t], dtype) : xr;
                float acc = bv;
                for (int k = 0; k < W; ++k) {
                    const int64_t src = t - (W - 1) + k;
                    float v = 0.0f;
                    if (src >= 0 && seq_idx[b * L + src] == seq_idx[b * L + t]) {
                        v = load_elem(x, row + src, dtype);
                        if (mask) v = round_to(v * mask[b * L + src], dtype);
                    }
                    acc = fmaf(w[k], v, acc);
                }
                if (use_silu) acc = silu(acc);
                if (residual_mode) acc += (residual_mode == 1) ? xm_t : xr;
                store_elem(out, row + t, dtype, acc);
            }
        }
    }
    return 0;
}

/*
 * Decode update, one token.  x, out [B, C]; conv_state [B, C, S] is updated
 * in place: shifted left by one with x appended (pure copies, so bit exact).
 *   out = act(bias + sum_{k<W-1} w[k] * state[S-(W-1)+k] + w[W-1] * x) (+ x)
 * round_mode 1 restates the eager step of model/model.py:385-396: every
 * product is rounded to the storage type, their fp32 sum is rounded, then
 * bias is added and rounded, then SiLU and rounded.
 */
int canon_oracle_update(const void *x, void *conv_state, const void *weight, const void *bias,
                        void *out, int64_t B, int64_t C, int W, int S,
                        int dtype, int w_dtype, int use_silu, int residual, int round_mode)
{
    if (W < 1 || W > 8 || S < 1 || S < W - 1 || B < 0 || C < 0) return -1;
    for (int64_t b = 0; b < B; ++b) {
        for (int64_t c = 0; c < C; ++c) {
            const int64_t r = b * C + c;
            float w[8], window[8];
            for (int k = 0; k < W; ++k) w[k] = round_to(load_elem(weight, c * W + k, w_dtype), dtype);
            const float bv = bias ? round_to(load_elem(bias, c, w_dtype), dtype) : 0.0f;
            const float xv = load_elem(x, r, dtype);
            for (int k = 0; k < W - 1; ++k)
                window[k] = load_elem(conv_state, r * S + (S - (W - 1) + k), dtype);
            window[W - 1] = xv;
            float acc;
            if (!round_mode) {
                acc = bv;
                for (int k = 0; k < W; ++k) acc = fmaf(w[k], window[k], acc);
                if (use_silu) acc = silu(acc);
                if (residual) acc += xv;
            } else {
                float s = 0.0f;
                for (int k = 0; k < W; ++k) s += round_to(window[k] * w[k], dtype);
                s = round_to(s, dtype);
                acc = round_to(bv + s, dtype);
                if (use_silu) acc = round_to(silu(acc), dtype);
                if (residual) acc = acc + xv;
            }
            store_elem(out, r, dtype, acc);
            /* shift left by one, append the new token: raw copies */
            const size_t es = (dtype == CANON_F32) ? 4 : 2;
            char *row = (char *)conv_state + (size_t)r * S * es;
            memmove(row, row + es, (size_t)(S - 1) * es);
            memcpy(row + (size_t)(S - 1) * es, (const char *)x + (size_t)r * es, es);
        }
    }
    return 0;
}

/*
 * Decode update with the two state-addressing modes of the upstream call
 * signature that the reference never uses (model/model.py:305-311 passes
 * neither; the signature slots are listed at causal_conv1d_mps/__init__.py:304-312):
 *   conv_state_indices[b]  row of conv_state (a pool of `rows` rows) used by batch entry b; an entry whose
 *                          index is negative or not below `rows` is skipped (upstream's padding slots):
 *                          no state row is touched and its row of out is left as it was
 *   cache_seqlens[b]       circular-buffer mode: the token is written to slot
 *                          cache_seqlens[b] % S, the W-1 slots before it
 *                          (cyclically) are the history, nothing is shifted
 * Fused rounding only.  PARITY UNPINNED against upstream (absent from the
 * reference tree); pinned by its equivalence with canon_oracle_update: the same
 * tokens fed with cache_seqlens = 0, 1, 2, .. give the same outputs, and the
 * buffer read cyclically from the write position is the shifted state.
 */
int canon_oracle_update_ext(const void *x, void *conv_state, const void *weight, const void *bias, void *out,
                            int64_t B, int64_t C, int W, int S, int dtype, int w_dtype, int use_silu,
                            int residual, const int32_t *cache_seqlens, const int32_t *conv_state_indices, int64_t rows)
{
    if (W < 1 || W > 8 || S < 1 || S < W - 1 || B < 0 || C < 0) return -1;
    const size_t es = (dtype == CANON_F32) ? 4 : 2;
    for (int64_t b = 0; b < B; ++b) {
        const int64_t srow = conv_state_indices ? conv_state_indices[b] : b;
        if (conv_state_indices && (srow < 0 || srow >= rows)) continue;
        for (int64_t c = 0; c < C; ++c) {
            const int64_t r = b * C + c, sr = srow * C + c;
            float w[8], window[8];
            for (int k = 0; k < W; ++k) w[k] = round_to(load_elem(weight, c * W + k, w_dtype), dtype);
            const float bv = bias ? round_to(load_elem(bias, c, w_dtype), dtype) : 0.0f;
            const float xv = load_elem(x, r, dtype);
            int pos = -1;
            if (cache_seqlens) pos = (int)(((cache_seqlens[b] % S) + S) % S);
            for (int k = 0; k < W - 1; ++k) {
                int slot = S - (W - 1) + k;
                if (pos >= 0) slot = ((pos - (W - 1) + k) % S + S) % S;
                window[k] = load_elem(conv_state, sr * S + slot, dtype);
            }
            window[W - 1] = xv;
            float acc = bv;
            for (int k = 0; k < W; ++k) acc = fmaf(w[k], window[k], acc);
            if (use_silu) acc = silu(acc);
            if (residual) acc += xv;
            store_elem(out, r, dtype, acc);
            char *row = (char *)conv_state + (size_t)sr * S * es;
            if (pos >= 0) {
                memcpy(row + (size_t)pos * es, (const char *)x + (size_t)r * es, es);
            } else {
                memmove(row, row + es, (size_t)(S - 1) * es);
                memcpy(row + (size_t)(S - 1) * es, (const char *)x + (size_t)r * es, es);
            }
        }
    }
    return 0;
}
