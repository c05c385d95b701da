// Kernel argument blocks, launch plans and launcher entry points shared by the
// translation units of libcanon_conv1d.so: canon_api.hip plans (pure host
// code), canon_fwd.hip / canon_update.hip / canon_bwd.hip hold the kernels and
// the functions that pick the template instance and launch it.
#ifndef CANON_PLAN_H
#define CANON_PLAN_H

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <string.h>

#include "canon_conv1d.h"

// build-time tuning knob of the channel-contiguous prefill kernel
#ifndef CANON_BLC_ROWS
#define CANON_BLC_ROWS 8
#endif

namespace canon {

// Division by a run-time constant as multiply-high and shifts (set up on the host).
struct FastDiv {
    uint32_t d, m, s1, s2;
};

// How a lane of the channel-contiguous kernels (prefill, decode update) gets its taps and bias.  The two common layouts are straight-line
// code (every load of the kernel is in flight before the first wait; the general path branches on the
// run-time weight type between its loads, which costs a wait per branch); which one runs is wave-uniform.
enum TapMode {
    TAPS_SAME,   // contiguous, 16-byte aligned [C, 4] weights of x's type (bias too, 4-byte aligned)
    TAPS_WIDE,   // the same with fp32 weights and bias and 16-bit x
    TAPS_ANY     // any strides, width and type
};

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
    int32_t W, w_dtype, mask_dtype, act, res_mode, eager, S_in, S_out, w_vec, b_pair, m_vec, nt, tap_mode;
    // launch geometry
    uint32_t nvec;      // bcl: vectors per row        blc: channel vectors per time row
    uint32_t nseg;      // bcl: segments per row       generic: time chunks per row     blc: groups of time tiles per sequence
    uint32_t chunk;     // generic: time steps per chunk                                 blc: time tiles per group
    uint32_t ntasks;    // bcl: wave tasks   blc: columns (batch x group x channel tile)   generic: threads
    uint32_t nblocks;   // blocks to launch
    FastDiv div_nseg, div_C;   // blc: div_nseg divides by `chunk`
    // blc: tiles
    uint32_t nct, ntt;  // channel tiles per row, time tiles per sequence
    FastDiv div_nct, div_ntt;   // div_ntt divides by the groups per sequence
    // two equal dense parts in one launch (canon_fwd_blc_pair_kernel): this is part 0's block, and what part 1 adds
    int64_t pair_out_shift;     // bytes from part 0's out to part 1's
    uint32_t pair_c;            // channels of a part: part 1's first channel in taps, bias, initial and final state
};

struct UpdArgs {
    // The fields the vectorised kernel reads on its usual path come first, within three 64-byte lines of the
    // kernel-argument segment: the kernel lives for a few microseconds, so every scalar-cache miss a wave
    // takes in turn before its first memory request shows in the total.
    const char *x;
    char *out;
    char *state;
    const void *weight;
    const void *bias;
    const void *tmask;
    uint32_t nthreads;
    uint32_t B;
    uint32_t nvec;      // lanes per batch row (channels / channels per lane)
    int32_t tap_mode;
    // second line
    int64_t x_sb, o_sb, s_sb, m_sb;
    FastDiv div_nvec;
    int32_t act, res_mode, mask_dtype, w_dtype;
    // third line: what the vectorised kernel reads off its usual path (state pool, general tap path)
    const int32_t *indices;   // conv_state row of batch entry b (state pool shared by many sequences)
    int64_t w_sc, w_sk;
    int32_t w_vec;
    uint32_t state_rows;      // rows of the state pool (0: not stated, indices are only checked for a negative value)
    // the rest: strided kernel, ring buffer, launch geometry
    const int32_t *seqlens;   // circular-buffer mode: conv_state is written at seqlens[b] % S, not shifted
    int64_t x_sc, o_sc;
    int64_t s_sc, s_ss;
    uint32_t C;
    int32_t W, S, eager;
    uint32_t bgroups;   // batch groups (each thread walks nb batch rows)
    uint32_t nb;
};
static_assert(offsetof(UpdArgs, x_sb) == 64 && offsetof(UpdArgs, indices) == 128 && offsetof(UpdArgs, x_sc) <= 192,
              "fields the vectorised update reads: three 64-byte lines");

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
    const int32_t *seq;   // packed-sequence indices [B, L] or nullptr (walk kernel only)
    int64_t q_sb, q_sl;
    const char *init;     // inputs before t = 0, [B, C, S_in], or nullptr (walk and channel-contiguous kernels)
    char *dinit;          // their gradient, or nullptr
    const char *dfin;     // gradient of the captured final state [B, C, S_out], or nullptr (same kernels)
    int64_t i_sb, i_sc, i_ss, j_sb, j_sc, j_ss, k_sb, k_sc, k_ss;
    int32_t S_in, S_out;
    int64_t x_sb, x_sc, x_sl;
    int64_t g_sb, g_sc, g_sl;
    int64_t d_sb, d_sc, d_sl;
    int64_t w_sc, w_sk;
    int64_t m_sb, m_sl;
    uint32_t B, C, L;
    int32_t W, w_dtype, mask_dtype, act, res_mode, w_vec, b_pair, m_vec;
    uint32_t nvec;      // channel groups per row (C / E)
    uint32_t nchunk;    // time chunks per sequence
    uint32_t chunk;     // time steps per chunk
    uint32_t nthreads;
    uint32_t nsets;     // partial sets = B * nchunk
    uint32_t nct;       // blc: channel tiles per row
    FastDiv div_nvec, div_nchunk, div_nct;
};

// backward of one decode step: a thread owns a channel and walks the batch entries of its group
struct UpdBwdArgs {
    const char *x;
    const char *state;     // the state before the step
    const char *dy;
    const char *dso;       // gradient w.r.t. the updated state, or nullptr
    char *dx;
    char *ds;              // gradient w.r.t. the state before, or nullptr
    const void *weight;
    const void *bias;
    const void *tmask;
    float *partial;        // [ngroups][C][5] partial sums of dweight / dbias, or nullptr
    float *dweight;
    float *dbias;
    int64_t x_sb, x_sc, g_sb, g_sc, d_sb, d_sc;
    int64_t s_sb, s_sc, s_ss, q_sb, q_sc, q_ss, r_sb, r_sc, r_ss;   // state, dstate_out, dstate
    int64_t w_sc, w_sk, m_sb;
    uint32_t B, C;
    uint32_t group;        // batch entries per group
    uint32_t ngroups;
    int32_t W, S, w_dtype, mask_dtype, act, res_mode;
    // the modes the strided kernel alone covers
    const int32_t *seqlens;   // ring buffer: the forward wrote the token to slot seqlens[b] % S
    const int32_t *indices;   // state pool: batch entry b used row indices[b] of the state tensors
    uint32_t state_rows;      // rows of the pool (0: not stated)
};

// Several channel ranges of one logical [B, C, L] problem that live in separate
// tensors (q / k / v or gate / up projections), one launch: every block belongs
// to one part and runs the single-tensor code on that part's argument block.
constexpr int kMaxParts = CANON_CONV1D_MAX_PARTS;

template <typename Args> struct PartTable {
    Args part[kMaxParts];
    uint32_t first_block[kMaxParts];   // first block of each part; 0xFFFFFFFF for unused slots
};

// ---------------------------------------------------------------------------
// kernel geometry (needed by the planner and by the kernels)
// ---------------------------------------------------------------------------
#ifndef CANON_BLC_WAVES
#define CANON_BLC_WAVES 4
#endif
constexpr int kBlcWaves = CANON_BLC_WAVES;   // time slabs per block
#ifndef CANON_BLC_WC
#define CANON_BLC_WC 1
#endif
constexpr int kBlcWC = CANON_BLC_WC;         // 64-lane channel tiles per block
constexpr int kBlcThreads = 64 * kBlcWaves * kBlcWC;
constexpr int kBlcGroup = 8;                 // most consecutive time tiles of a channel tile that follow each other on one XCD
constexpr int kBlcVecBytes = 8;   // bytes per lane and access: 8 measured 4-9 % faster than 16 (half the registers, twice the waves)
#ifndef CANON_BWD_SLAB
#define CANON_BWD_SLAB 8
#endif
constexpr int kBwdSlab = CANON_BWD_SLAB;    // time steps per wave and tile
#ifndef CANON_BWD_VEC_BYTES
#define CANON_BWD_VEC_BYTES 8
#endif
constexpr int kBwdVecBytes = CANON_BWD_VEC_BYTES;   // bytes per lane and row in the channel-contiguous backward
constexpr int kBwdWaves = 4;
constexpr int kBwdMaxChunk = 32 * kBwdSlab * kBwdWaves;   // most time steps one block of the channel-contiguous backward walks
enum FwdKind { FWD_BCL, FWD_BCL_SHORT, FWD_BLC, FWD_GENERIC };
#ifndef CANON_BCL_MAX_U
#define CANON_BCL_MAX_U 4
#endif
constexpr int kBclMaxVectorsPerLane = CANON_BCL_MAX_U;   // most 16-byte vectors a lane of the time-contiguous kernel takes (1, 2 or 4)
enum UpdKind { UPD_VEC, UPD_GENERIC };

constexpr uint32_t kGenericChunk = 8;   // time steps per thread in the scalar kernel
constexpr int kBlcRows = CANON_BLC_ROWS;   // time steps per wave in the channel-contiguous kernel
// ... and in its unmasked width-4 launches that move at least kBlcShortSlabBytes (single tensor or pair): measured
// 2-8 % faster there (B 8, C 3456, bf16: 19.9 -> 19.45 us, with SiLU 20.85 -> 19.86 us; B 16, C 640: 10.2 -> 9.4 us),
// 5-16 % slower below that size (B 8, C 640 / 960: 5.3 -> 6.2 / 6.7 -> 7.8 us) and 0-4 % slower with a padding mask
#ifndef CANON_BLC_ROWS_SHORT
#define CANON_BLC_ROWS_SHORT 4
#endif
constexpr int kBlcRowsShort = CANON_BLC_ROWS_SHORT;
constexpr uint64_t kBlcShortSlabBytes = 40ull << 20;
constexpr uint64_t kStreamBytes = 64ull << 20;  // above this much traffic, x / out are accessed non-temporally
constexpr int kUpdNB = 2;               // batch rows per lane in the vectorised update when there is plenty of work
// channels a lane of the vectorised update owns: as many as make its piece of the [B, C, S] state one run
// of 12 or 16 bytes (fp32 with 8 slots: 32)
constexpr int upd_lane_channels(int elem_bytes, int S) { return (elem_bytes == 2 && S != 8) ? 2 : 1; }
enum BwdKind { BWD_BLC_VEC, BWD_BCL_VEC, BWD_GENERIC };
constexpr int kBwdRows = 4;   // rows fetched ahead per lane in the backward walk
#ifndef CANON_BWD_HALF_BLOCKS
#define CANON_BWD_HALF_BLOCKS 3
#endif
constexpr int kBwdHalfBlocksPerCU = CANON_BWD_HALF_BLOCKS;   // grid target of the channel-contiguous backward, in half blocks per CU

// ---------------------------------------------------------------------------
// launch plans: what the validated arguments of one call turn into
// ---------------------------------------------------------------------------
// waves per block of the time-contiguous prefill: 4, or 8 in unmasked launches of at least kBclBigLaunch waves (64
// per CU); with a mask 1 (blocks of 8 measured 6-9 % slower, of 1 1-2 % faster than of 4)
constexpr int kBclMaxWaves = 8;
constexpr uint32_t kBclBigLaunch = 16384;

struct FwdPlan {
    FwdKind kind;
    int U;
    bool edge;   // bcl: rows do not start on 16-byte boundaries
    uint32_t wpb; // bcl: waves per block
    int rows;    // blc: time steps per wave (kBlcRows or kBlcRowsShort)
    FwdArgs args;
    uint32_t grid;
};

struct UpdPlan {
    UpdKind kind;
    UpdArgs args;
    uint32_t grid;
};

struct FwdPartsPlan {
    int n;
    bool single;            // one launch over a PartTable
    bool pair;              // ... or, two equal dense parts, one launch of the pair kernel on part[0]'s block
    uint32_t grid;          // of that launch
    FwdPlan part[kMaxParts];
};

struct UpdPartsPlan {
    int n;
    bool single;
    uint32_t grid;
    UpdPlan part[kMaxParts];
};

struct BwdPlan {
    BwdKind kind;
    int U;
    BwdArgs args;
    uint32_t grid;
    int64_t workspace_bytes;
};

struct UpdBwdPlan {
    bool vec;               // contiguous states of 3 or 4 slots, channel-contiguous token: dense 4 / 12 / 16-byte lanes
    UpdBwdArgs args;
    uint32_t grid_c;        // blocks along the channels (0: nothing to launch)
    int64_t workspace_bytes;
};

// Launchers (x_dtype is a CANON_DTYPE_* code; nothing here synchronises)
void launch_fwd(const FwdPlan &pl, int x_dtype, hipStream_t s);
void launch_fwd_parts(const FwdPartsPlan &pp, int x_dtype, hipStream_t s);
void launch_update(const UpdPlan &pl, int x_dtype, hipStream_t s);
void launch_update_parts(const UpdPartsPlan &pp, int x_dtype, hipStream_t s);
void launch_bwd(const BwdPlan &pl, int x_dtype, hipStream_t s);          // dx + partial sets, then the reduction
void launch_update_bwd(const UpdBwdPlan &pl, int x_dtype, hipStream_t s);   // dx, dstate + partial sets, then the reduction
void launch_zero(float *p, uint32_t n, hipStream_t s);                    // fill kernel (graph-capture safe)
// Make the runtime load this translation unit's code object onto the current device now (it would otherwise do so
// at the unit's first launch): hipSuccess or the runtime's error.
hipError_t preload_fwd();
hipError_t preload_update();
hipError_t preload_bwd();

}  // namespace canon
#endif  // CANON_PLAN_H
