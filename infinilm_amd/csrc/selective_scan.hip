// A selective scan whose decay is a matrix: every channel c keeps `state` numbers of its own,
//
//   dt_c = softplus(raw_c + bias_c)
//   S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n,   A = -exp(A_log)        (per token, from the request's state row)
//   y_c = sum_n S[c, n] C_n + D_c x_c,   out_c = y_c * silu(z_c)
//
// with x (after its convolution and activation) in float32, the raw step sizes, B, C and z in the activations' dtype.
// Everything that enters the recurrence is float32: step sizes, softplus, exponentials, the state, the sums.
//
// A channel's state lies across 16 lanes (entry n in lane n % 16, R = ceil(state / 16) registers a lane); a block of 256
// threads takes 16 channels of one request and walks its tokens in order, the next token's operands on their way while
// this one is computed.  The state passes from step to step through the request's pool row [inner, state], so the
// result does not depend on how a prompt is cut.
#include "common.h"

__device__ __forceinline__ float ss_softplus(float v) { return v > 20.f ? v : log1pf(expf(v)); }

template <typename T, typename TW, int R>
__global__ void __launch_bounds__(256)
selective_scan_kernel(T* __restrict__ out, int out_stride, const float* __restrict__ x, int x_stride, const T* __restrict__ raw,
                      int raw_stride, const TW* __restrict__ dt_bias, const T* __restrict__ B, const T* __restrict__ C, int bc_stride,
                      const T* __restrict__ z, int z_stride, const float* __restrict__ a_log, const float* __restrict__ skip,
                      float* __restrict__ pool, const int* __restrict__ state_in, const int* __restrict__ state_out,
                      const int* __restrict__ seg_offsets, int inner, int state) {
    const int sgm = blockIdx.y;
    const int c = blockIdx.x * 16 + (threadIdx.x >> 4), sub = threadIdx.x & 15;
    const int t0 = seg_offsets[sgm], t1 = seg_offsets[sgm + 1];
    if (c >= inner || t0 >= t1) return;
    const int row_in = state_in[sgm], row_out = state_out[sgm];
    float S[R], A[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int n = sub + 16 * r;
        const bool ok = n < state;
        S[r] = ok ? pool[((size_t)row_in * inner + c) * state + n] : 0.f;
        A[r] = ok ? -expf(a_log[(size_t)c * state + n]) : 0.f;
    }
    const float bias = to_f32(dt_bias[c]), Dc = skip[c];
    // the first token's operands
    float xv = x[(size_t)t0 * x_stride + c], rv = to_f32(raw[(size_t)t0 * raw_stride + c]), zv = to_f32(z[(size_t)t0 * z_stride + c]);
    float Bv[R], Cv[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int n = sub + 16 * r;
        Bv[r] = n < state ? to_f32(B[(size_t)t0 * bc_stride + n]) : 0.f;
        Cv[r] = n < state ? to_f32(C[(size_t)t0 * bc_stride + n]) : 0.f;
    }
    for (int t = t0; t < t1; ++t) {
        const int tn = t + 1 < t1 ? t + 1 : t;       // the next token's operands (the last token's again at the end)
        const float xn = x[(size_t)tn * x_stride + c], rn = to_f32(raw[(size_t)tn * raw_stride + c]), zn = to_f32(z[(size_t)tn * z_stride + c]);
        float Bn[R], Cn[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int n = sub + 16 * r;
            Bn[r] = n < state ? to_f32(B[(size_t)tn * bc_stride + n]) : 0.f;
            Cn[r] = n < state ? to_f32(C[(size_t)tn * bc_stride + n]) : 0.f;
        }
        const float dt = ss_softplus(rv + bias);
        const float dx = dt * xv;
        float y = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            S[r] = fmaf(expf(dt * A[r]), S[r], dx * Bv[r]);
            y = fmaf(S[r], Cv[r], y);
        }
        y += __shfl_xor(y, 8, 64);
        y += __shfl_xor(y, 4, 64);
        y += __shfl_xor(y, 2, 64);
        y += __shfl_xor(y, 1, 64);
        if (sub == 0) {
            y = fmaf(Dc, xv, y);
            out[(size_t)t * out_stride + c] = from_f32<T>(y * (zv / (1.0f + expf(-zv))));
        }
        xv = xn; rv = rn; zv = zn;
#pragma unroll
        for (int r = 0; r < R; ++r) { Bv[r] = Bn[r]; Cv[r] = Cn[r]; }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int n = sub + 16 * r;
        if (n < state) pool[((size_t)row_out * inner + c) * state + n] = S[r];
    }
}

extern "C" int ilm_selective_scan_max_state() { return 256; }

// out [T, inner]; x float32 [T, inner]; raw, z [T, inner]; B, C [T, state] (rows of one stride); a_log [inner, state] and
// skip [inner] float32; pool float32 [rows, inner, state]; segment r covers rows seg_offsets[r] .. seg_offsets[r + 1] - 1
extern "C" int ilm_selective_scan(void* out, int out_stride, const void* x, int x_stride, const void* raw, int raw_stride,
                                  const void* dt_bias, const void* B, const void* C, int bc_stride, const void* z, int z_stride,
                                  const void* a_log, const void* skip, void* pool, const void* state_in, const void* state_out,
                                  const void* seg_offsets, int segments, int inner, int state, int dtype, int w_dt, hipStream_t stream) {
    ILM_REQUIRE(segments > 0 && segments <= 65535 && inner > 0 && state > 0, "selective_scan: bad sizes");
    ILM_REQUIRE(state <= ilm_selective_scan_max_state(), "selective_scan: %d state entries a channel (at most %d)", state,
                ilm_selective_scan_max_state());
    ILM_REQUIRE(out_stride >= inner && x_stride >= inner && raw_stride >= inner && z_stride >= inner && bc_stride >= state,
                "selective_scan: rows shorter than their channels");
    dim3 grid((inner + 15) / 16, segments);
#define SS_ARGS(T__, TW__) (T__*)out, out_stride, (const float*)x, x_stride, (const T__*)raw, raw_stride, (const TW__*)dt_bias,       \
                           (const T__*)B, (const T__*)C, bc_stride, (const T__*)z, z_stride, (const float*)a_log, (const float*)skip, \
                           (float*)pool, (const int*)state_in, (const int*)state_out, (const int*)seg_offsets, inner, state
#define SS_BY_R(T__, TW__)                                                                                      \
    {                                                                                                           \
        const int regs = (state + 15) / 16;                                                                     \
        if (regs <= 1) selective_scan_kernel<T__, TW__, 1><<<grid, 256, 0, stream>>>(SS_ARGS(T__, TW__));        \
        else if (regs <= 2) selective_scan_kernel<T__, TW__, 2><<<grid, 256, 0, stream>>>(SS_ARGS(T__, TW__));   \
        else if (regs <= 4) selective_scan_kernel<T__, TW__, 4><<<grid, 256, 0, stream>>>(SS_ARGS(T__, TW__));   \
        else if (regs <= 8) selective_scan_kernel<T__, TW__, 8><<<grid, 256, 0, stream>>>(SS_ARGS(T__, TW__));   \
        else selective_scan_kernel<T__, TW__, 16><<<grid, 256, 0, stream>>>(SS_ARGS(T__, TW__));                 \
    }
    if (dtype == ILM_DTYPE_F32 && w_dt == ILM_DTYPE_F32) SS_BY_R(float, float)
    else if (dtype == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_BF16) SS_BY_R(bf16, bf16)
    else if (dtype == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_F32) SS_BY_R(bf16, float)
    else ILM_REQUIRE(false, "selective_scan: dtypes %d / %d", dtype, w_dt);
#undef SS_BY_R
#undef SS_ARGS
    ILM_LAUNCH_CHECK("selective_scan");
    return 0;
}
