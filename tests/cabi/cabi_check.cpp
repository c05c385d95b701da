// The C ABI used the way a C++ host (a serving runtime that owns its buffers) would use it: no
// Python, no framework types.  Runs a Canon-D sized prefill with padding mask, bias, residual and
// conv-state capture on channel-contiguous bf16 tensors, then carries the captured state through
// decode steps -- eagerly and as a captured HIP graph -- and compares every byte with the CPU
// oracle (oracle/libcanon_oracle.so, test infrastructure).
//
//   usage: cabi_check <path to libcanon_oracle.so>
#include <dlfcn.h>
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <vector>

#include "canon_conv1d.h"

#define CK(x)                                                                              \
    do {                                                                                   \
        hipError_t e_ = (x);                                                               \
        if (e_ != hipSuccess) {                                                            \
            printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);          \
            return 2;                                                                      \
        }                                                                                  \
    } while (0)
#define CANON(x)                                                                           \
    do {                                                                                   \
        if ((x) != CANON_OK) {                                                             \
            printf("library error at line %d: %s\n", __LINE__, canon_conv1d_last_error()); \
            return 3;                                                                      \
        }                                                                                  \
    } while (0)

typedef int (*oracle_fwd_t)(const void *, const void *, const void *, const float *, const void *, void *, void *, int64_t,
                            int64_t, int64_t, int, int, int, int, int, int, int, int);
typedef int (*oracle_update_t)(const void *, void *, const void *, const void *, void *, int64_t, int64_t, int, int, int,
                               int, int, int, int);
typedef uint16_t (*to_bf16_t)(float);

static uint32_t rng_state = 12345u;
static float next_uniform()   // xorshift, (-1, 1)
{
    rng_state ^= rng_state << 13;
    rng_state ^= rng_state >> 17;
    rng_state ^= rng_state << 5;
    return (float)(rng_state >> 8) / 8388608.0f - 1.0f;
}

static int count_diff(const std::vector<uint16_t> &a, const std::vector<uint16_t> &b)
{
    int n = 0;
    for (size_t i = 0; i < a.size(); ++i) n += a[i] != b[i];
    return n;
}

int main(int argc, char **argv)
{
    if (argc < 2) {
        printf("usage: %s <libcanon_oracle.so>\n", argv[0]);
        return 1;
    }
    void *h = dlopen(argv[1], RTLD_NOW);
    if (!h) {
        printf("cannot load the oracle: %s\n", dlerror());
        return 1;
    }
    oracle_fwd_t oracle_fwd = (oracle_fwd_t)dlsym(h, "canon_oracle_fwd");
    oracle_update_t oracle_update = (oracle_update_t)dlsym(h, "canon_oracle_update");
    to_bf16_t to_bf16 = (to_bf16_t)dlsym(h, "canon_oracle_float_to_bf16");
    if (!oracle_fwd || !oracle_update || !to_bf16) {
        printf("oracle symbols missing\n");
        return 1;
    }
    if (canon_conv1d_abi_version() != CANON_CONV1D_ABI_VERSION) {
        printf("header / library ABI mismatch\n");
        return 1;
    }

    const int64_t B = 3, C = 1728, L = 200, S = 8;
    const int W = 4, steps = 6;
    // host data, logical [B, C, L]; the device copy is channel-contiguous ([B, L, C])
    std::vector<uint16_t> x_bcl(B * C * L), x_blc(B * L * C), w(C * W), bias(C), tok(steps * B * C);
    std::vector<float> mask_f(B * L);
    std::vector<int64_t> mask_i(B * L);
    for (auto &v : x_bcl) v = to_bf16(next_uniform() * 2.0f);
    for (auto &v : w) v = to_bf16(next_uniform() * 0.5f);
    for (auto &v : bias) v = to_bf16(next_uniform() * 0.2f);
    for (auto &v : tok) v = to_bf16(next_uniform() * 2.0f);
    const int64_t valid[3] = {200, 77, 5};
    for (int64_t b = 0; b < B; ++b)
        for (int64_t t = 0; t < L; ++t) {
            mask_i[b * L + t] = t < valid[b];
            mask_f[b * L + t] = (float)mask_i[b * L + t];
        }
    for (int64_t b = 0; b < B; ++b)
        for (int64_t c = 0; c < C; ++c)
            for (int64_t t = 0; t < L; ++t) x_blc[(b * L + t) * C + c] = x_bcl[(b * C + c) * L + t];

    // ---- oracle ----------------------------------------------------------------------------
    std::vector<uint16_t> want_bcl(B * C * L), want_state(B * C * S);
    if (oracle_fwd(x_bcl.data(), w.data(), bias.data(), mask_f.data(), nullptr, want_bcl.data(), want_state.data(), B, C, L,
                   W, 0, (int)S, CANON_DTYPE_BF16, CANON_DTYPE_BF16, 0, CANON_RESIDUAL_MASKED, CANON_ROUND_FUSED)) {
        printf("oracle rejected the prefill\n");
        return 1;
    }
    std::vector<uint16_t> state_ref = want_state, want_tok_out(steps * B * C);
    std::vector<std::vector<uint16_t>> want_states;
    for (int i = 0; i < steps; ++i) {
        if (oracle_update(tok.data() + (size_t)i * B * C, state_ref.data(), w.data(), bias.data(),
                          want_tok_out.data() + (size_t)i * B * C, B, C, W, (int)S, CANON_DTYPE_BF16, CANON_DTYPE_BF16, 0, 1,
                          CANON_ROUND_FUSED)) {
            printf("oracle rejected the update\n");
            return 1;
        }
        want_states.push_back(state_ref);
    }

    // ---- device ----------------------------------------------------------------------------
    void *d_x, *d_out, *d_w, *d_bias, *d_mask, *d_state, *d_tok, *d_tok_out;
    CK(hipMalloc(&d_x, x_blc.size() * 2));
    CK(hipMalloc(&d_out, x_blc.size() * 2));
    CK(hipMalloc(&d_w, w.size() * 2));
    CK(hipMalloc(&d_bias, bias.size() * 2));
    CK(hipMalloc(&d_mask, mask_i.size() * 8));
    CK(hipMalloc(&d_state, want_state.size() * 2));
    CK(hipMalloc(&d_tok, tok.size() * 2));
    CK(hipMalloc(&d_tok_out, tok.size() * 2));
    CK(hipMemcpy(d_x, x_blc.data(), x_blc.size() * 2, hipMemcpyHostToDevice));
    CK(hipMemcpy(d_w, w.data(), w.size() * 2, hipMemcpyHostToDevice));
    CK(hipMemcpy(d_bias, bias.data(), bias.size() * 2, hipMemcpyHostToDevice));
    CK(hipMemcpy(d_mask, mask_i.data(), mask_i.size() * 8, hipMemcpyHostToDevice));
    CK(hipMemcpy(d_tok, tok.data(), tok.size() * 2, hipMemcpyHostToDevice));
    hipStream_t stream;
    CK(hipStreamCreate(&stream));

    canon_conv1d_fwd_params f;
    memset(&f, 0, sizeof f);
    f.struct_size = sizeof f;
    f.x_dtype = f.w_dtype = CANON_DTYPE_BF16;
    f.mask_dtype = CANON_MASK_I64;
    f.width = W;
    f.residual_mode = CANON_RESIDUAL_MASKED;
    f.batch = B; f.channels = C; f.seqlen = L;
    f.x = d_x; f.x_stride_b = L * C; f.x_stride_c = 1; f.x_stride_l = C;
    f.out = d_out; f.out_stride_b = L * C; f.out_stride_c = 1; f.out_stride_l = C;
    f.weight = d_w; f.w_stride_c = W; f.w_stride_k = 1;
    f.bias = d_bias;
    f.mask = d_mask; f.mask_stride_b = L; f.mask_stride_l = 1;
    f.final_state = d_state; f.final_len = (int)S;
    f.final_stride_b = C * S; f.final_stride_c = S; f.final_stride_s = 1;
    const char *plan = canon_conv1d_fwd_plan(&f);
    if (!plan || strcmp(plan, "blc_vec") != 0) {
        printf("prefill planned as %s, expected blc_vec\n", plan ? plan : "(rejected)");
        return 1;
    }
    CANON(canon_conv1d_fwd(&f, stream));
    CK(hipStreamSynchronize(stream));
    std::vector<uint16_t> got_blc(x_blc.size()), got_state(want_state.size());
    CK(hipMemcpy(got_blc.data(), d_out, got_blc.size() * 2, hipMemcpyDeviceToHost));
    CK(hipMemcpy(got_state.data(), d_state, got_state.size() * 2, hipMemcpyDeviceToHost));
    int bad = 0;
    for (int64_t b = 0; b < B; ++b)
        for (int64_t c = 0; c < C; ++c)
            for (int64_t t = 0; t < L; ++t) bad += got_blc[(b * L + t) * C + c] != want_bcl[(b * C + c) * L + t];
    printf("prefill %s: %d of %zu outputs differ, %d of %zu state entries differ\n", plan, bad, got_blc.size(),
           count_diff(got_state, want_state), got_state.size());
    if (bad || count_diff(got_state, want_state)) return 4;

    // ---- decode steps, eagerly --------------------------------------------------------------
    std::vector<canon_conv1d_update_params> u(steps);
    for (int i = 0; i < steps; ++i) {
        canon_conv1d_update_params &p = u[i];
        memset(&p, 0, sizeof p);
        p.struct_size = sizeof p;
        p.x_dtype = p.w_dtype = CANON_DTYPE_BF16;
        p.width = W; p.state_len = (int)S; p.residual_mode = CANON_RESIDUAL_MASKED;
        p.batch = B; p.channels = C;
        p.x = (char *)d_tok + (size_t)i * B * C * 2; p.x_stride_b = C; p.x_stride_c = 1;
        p.out = (char *)d_tok_out + (size_t)i * B * C * 2; p.out_stride_b = C; p.out_stride_c = 1;
        p.conv_state = d_state; p.state_stride_b = C * S; p.state_stride_c = S; p.state_stride_s = 1;
        p.weight = d_w; p.w_stride_c = W; p.w_stride_k = 1;
        p.bias = d_bias;
    }
    const char *uplan = canon_conv1d_update_plan(&u[0]);
    if (!uplan || strcmp(uplan, "update_vec") != 0) {
        printf("update planned as %s, expected update_vec\n", uplan ? uplan : "(rejected)");
        return 1;
    }
    std::vector<uint16_t> got_tok_out(tok.size());
    for (int i = 0; i < steps; ++i) CANON(canon_conv1d_update(&u[i], stream));
    CK(hipStreamSynchronize(stream));
    CK(hipMemcpy(got_tok_out.data(), d_tok_out, got_tok_out.size() * 2, hipMemcpyDeviceToHost));
    CK(hipMemcpy(got_state.data(), d_state, got_state.size() * 2, hipMemcpyDeviceToHost));
    printf("decode, %d eager steps: %d outputs differ, %d state entries differ\n", steps, count_diff(got_tok_out, want_tok_out),
           count_diff(got_state, want_states[steps - 1]));
    if (count_diff(got_tok_out, want_tok_out) || count_diff(got_state, want_states[steps - 1])) return 5;

    // ---- the same steps as one captured HIP graph, replayed twice from the prefill's state -----
    hipGraph_t graph;
    hipGraphExec_t exec;
    CK(hipStreamBeginCapture(stream, hipStreamCaptureModeGlobal));
    for (int i = 0; i < steps; ++i) CANON(canon_conv1d_update(&u[i], stream));
    CK(hipStreamEndCapture(stream, &graph));
    CK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
    for (int replay = 0; replay < 2; ++replay) {
        CK(hipMemcpy(d_state, want_state.data(), want_state.size() * 2, hipMemcpyHostToDevice));
        CK(hipMemset(d_tok_out, 0xFF, tok.size() * 2));
        CK(hipDeviceSynchronize());
        CK(hipGraphLaunch(exec, stream));
        CK(hipStreamSynchronize(stream));
        CK(hipMemcpy(got_tok_out.data(), d_tok_out, got_tok_out.size() * 2, hipMemcpyDeviceToHost));
        CK(hipMemcpy(got_state.data(), d_state, got_state.size() * 2, hipMemcpyDeviceToHost));
        const int d1 = count_diff(got_tok_out, want_tok_out), d2 = count_diff(got_state, want_states[steps - 1]);
        printf("decode, graph replay %d: %d outputs differ, %d state entries differ\n", replay, d1, d2);
        if (d1 || d2) return 6;
    }
    CK(hipGraphExecDestroy(exec));
    CK(hipGraphDestroy(graph));

    // ---- an invalid call reports through the status code, never through an exception ---------
    canon_conv1d_fwd_params badp = f;
    badp.width = 7;
    if (canon_conv1d_fwd(&badp, stream) != CANON_ERR_UNSUPPORTED || !strstr(canon_conv1d_last_error(), "width 7")) {
        printf("width 7 was not rejected as unsupported\n");
        return 7;
    }
    printf("cabi_check: OK\n");
    return 0;
}
