// A selective scan whose decay is a matrix: every channel c keeps `state` numbers of its own,
//
//   dt_c = softplus(raw_c + bias_c)
//   S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n,   A = -exp(A_log)        (per token, from the request's state row)
//   y_c = sum_n S[c, n] C_n + D_c x_c,   out_c = y_c * silu(z_c)
//
// with x (after its convolution and activation) in float32, the raw step sizes, B, C and z in the activations' dtype.
// Everything that enters the recurrence is float32: step sizes, softplus, exponentials, the state, the sums.
//
// Two forms.  States of up to 32 entries of at least 256 channels: a thread a channel (see below).  Otherwise a
// channel's state lies across 16 lanes (entry n in lane n % 16, R = ceil(state / 16) registers a lane); a block of 256
// threads takes 16 CH channels of one request (CH channels a lane group, their loads in flight together) and walks its
// tokens in order, the next token's operands on their way while this one is computed.  The state passes from step to step
// through the request's pool row [inner, state], so the result does not depend on how a prompt is cut.
//
// Long segments run in pieces of `piece` tokens side by side, in three launches: every piece from a zero state (its end
// state and the sum of its step sizes: a piece's decay is exp(A[c, n] sum dt_c)); the pieces' true start states, piece after
// piece, from the request's row (which then receives the segment's end state); every piece again from its start state, with
// the outputs.  Twice the arithmetic, a piece's length instead of the segment's as the chain; the sums are formed in another
// order than in one pass (float rounding).
#include "common.h"

__device__ __forceinline__ float ss_softplus(float v) { return v > 20.f ? v : log1pf(expf(v)); }

// pieces before segment `sgm` (every segment is cut from its own first token)
__device__ __forceinline__ int ss_piece_base(const int* seg_offsets, int sgm, int piece) {
    int base = 0;
    for (int r = 0; r < sgm; ++r) base += (seg_offsets[r + 1] - seg_offsets[r] + piece - 1) / piece;
    return base;
}

// MODE 0: the whole segment in one pass.  MODE 1: a piece from zero, no outputs; its end state and the sum of its step
// sizes go to the workspace.  MODE 2: a piece from its start state in the workspace, with outputs.
template <typename T, typename TW, int R, int CH, int MODE>
__global__ void __launch_bounds__(256)
selective_scan_kernel(T* __restrict__ out, int out_stride, const float* __restrict__ x, int x_stride, const T* __restrict__ raw,
                      int raw_stride, const TW* __restrict__ dt_bias, const T* __restrict__ B, const T* __restrict__ C, int bc_stride,
                      const T* __restrict__ z, int z_stride, const float* __restrict__ a_log, const float* __restrict__ skip,
                      float* __restrict__ pool, const int* __restrict__ state_in, const int* __restrict__ state_out,
                      const int* __restrict__ seg_offsets, int inner, int state, int piece, float* __restrict__ ws_state,
                      float* __restrict__ ws_dt) {
    const int sgm = blockIdx.y;
    const int c0 = (blockIdx.x * 16 + (threadIdx.x >> 4)) * CH, sub = threadIdx.x & 15;
    int t0 = seg_offsets[sgm], t1 = seg_offsets[sgm + 1];
    if (c0 >= inner || t0 >= t1) return;
    size_t slot = 0;
    if (MODE != 0) {
        const int first = t0 + (int)blockIdx.z * piece;
        if (first >= t1) return;
        slot = (size_t)ss_piece_base(seg_offsets, sgm, piece) + blockIdx.z;
        t0 = first;
        t1 = min(t1, first + piece);
    }
    const int row_in = state_in[sgm], row_out = state_out[sgm];
    float S[CH][R], A[CH][R], bias[CH], Dc[CH], dsum[CH];
    bool live[CH];
#pragma unroll
    for (int k = 0; k < CH; ++k) {
        const int c = c0 + k;
        live[k] = c < inner;
        const int cc = live[k] ? c : c0;
        bias[k] = to_f32(dt_bias[cc]);
        Dc[k] = skip[cc];
        dsum[k] = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int n = sub + 16 * r;
            const bool ok = n < state;
            const float* src = MODE == 0 ? pool + ((size_t)row_in * inner + cc) * state : ws_state + (slot * inner + cc) * state;
            S[k][r] = (ok && MODE != 1) ? src[n] : 0.f;
            A[k][r] = ok ? -expf(a_log[(size_t)cc * state + n]) : 0.f;
        }
    }
    // the first token's operands
    float xv[CH], rv[CH], zv[CH], Bv[R], Cv[R];
#pragma unroll
    for (int k = 0; k < CH; ++k) {
        const int cc = live[k] ? c0 + k : c0;
        xv[k] = x[(size_t)t0 * x_stride + cc];
        rv[k] = to_f32(raw[(size_t)t0 * raw_stride + cc]);
        zv[k] = MODE == 1 ? 0.f : to_f32(z[(size_t)t0 * z_stride + cc]);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int n = sub + 16 * r;
        Bv[r] = n < state ? to_f32(B[(size_t)t0 * bc_stride + n]) : 0.f;
        Cv[r] = (n < state && MODE != 1) ? to_f32(C[(size_t)t0 * bc_stride + n]) : 0.f;
    }
    for (int t = t0; t < t1; ++t) {
        const int tn = t + 1 < t1 ? t + 1 : t;       // the next token's operands (the last token's again at the end)
        float xn[CH], rn[CH], zn[CH], Bn[R], Cn[R];
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            const int cc = live[k] ? c0 + k : c0;
            xn[k] = x[(size_t)tn * x_stride + cc];
            rn[k] = to_f32(raw[(size_t)tn * raw_stride + cc]);
            zn[k] = MODE == 1 ? 0.f : to_f32(z[(size_t)tn * z_stride + cc]);
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int n = sub + 16 * r;
            Bn[r] = n < state ? to_f32(B[(size_t)tn * bc_stride + n]) : 0.f;
            Cn[r] = (n < state && MODE != 1) ? to_f32(C[(size_t)tn * bc_stride + n]) : 0.f;
        }
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            const float dt = ss_softplus(rv[k] + bias[k]);
            const float dx = dt * xv[k];
            dsum[k] += dt;
            float y = 0.f;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                S[k][r] = fmaf(expf(dt * A[k][r]), S[k][r], dx * Bv[r]);
                y = fmaf(S[k][r], Cv[r], y);
            }
            if (MODE != 1) {
                y += __shfl_xor(y, 8, 64);
                y += __shfl_xor(y, 4, 64);
                y += __shfl_xor(y, 2, 64);
                y += __shfl_xor(y, 1, 64);
                if (sub == 0 && live[k]) {
                    y = fmaf(Dc[k], xv[k], y);
                    out[(size_t)t * out_stride + c0 + k] = from_f32<T>(y * (zv[k] / (1.0f + expf(-zv[k]))));
                }
            }
            xv[k] = xn[k]; rv[k] = rn[k]; zv[k] = zn[k];
        }
#pragma unroll
        for (int r = 0; r < R; ++r) { Bv[r] = Bn[r]; Cv[r] = Cn[r]; }
    }
    if (MODE == 2) return;
#pragma unroll
    for (int k = 0; k < CH; ++k) {
        if (!live[k]) continue;
        float* dst = MODE == 0 ? pool + ((size_t)row_out * inner + c0 + k) * state : ws_state + (slot * inner + c0 + k) * state;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int n = sub + 16 * r;
            if (n < state) dst[n] = S[k][r];
        }
        if (MODE == 1 && sub == 0) ws_dt[slot * inner + c0 + k] = dsum[k];
    }
}

// States of up to 32 entries: a thread a channel with all its entries in registers (no exchange between lanes; step size,
// softplus and gate once a channel and token); a block takes 256 channels of one request (or of one piece of it), and a
// tile of 16 tokens' B and C rows lies in LDS, read by every thread at the same address.  Decays as exp2(dt A log2 e).
#define SC_TT 16
template <typename T, typename TW, int N, int MODE>
__global__ void __launch_bounds__(256)
selective_scan_channel_kernel(T* __restrict__ out, int out_stride, const float* __restrict__ x, int x_stride, const T* __restrict__ raw,
                              int raw_stride, const TW* __restrict__ dt_bias, const T* __restrict__ B, const T* __restrict__ C,
                              int bc_stride, const T* __restrict__ z, int z_stride, const float* __restrict__ a_log,
                              const float* __restrict__ skip, float* __restrict__ pool, const int* __restrict__ state_in,
                              const int* __restrict__ state_out, const int* __restrict__ seg_offsets, int inner, int state, int piece,
                              float* __restrict__ ws_state, float* __restrict__ ws_dt) {
    __shared__ float Bs[SC_TT][N], Cs[SC_TT][N];
    const int sgm = blockIdx.y, tid = threadIdx.x;
    const int c = blockIdx.x * 256 + tid;
    int t0 = seg_offsets[sgm], t1 = seg_offsets[sgm + 1];
    if (t0 >= t1) return;                                    // (the same for the whole block, as is the piece's test below)
    size_t slot = 0;
    if (MODE != 0) {
        const int first = t0 + (int)blockIdx.z * piece;
        if (first >= t1) return;
        slot = (size_t)ss_piece_base(seg_offsets, sgm, piece) + blockIdx.z;
        t0 = first;
        t1 = min(t1, first + piece);
    }
    const bool active = c < inner;
    const int cc = active ? c : inner - 1;
    // The block's 256 channels x state entries are one contiguous run of a state row (and of A_log): they pass through LDS in
    // whole lines, and every thread then takes its channel's entries from there (rows padded by one against bank conflicts).
    __shared__ float stage[256 * (N + 1)];
    float S[N], A2[N];
    const int ch0 = blockIdx.x * 256, run = min(256, inner - ch0) * state;
    // every load that does not depend on another is issued before the first barrier: the state's run and A_log's (element
    // tid + 256 j of the run), the first token's operands, the channel's constants
    const float* src = (MODE == 0 ? pool + (size_t)state_in[sgm] * inner * state : ws_state + slot * inner * state) + (size_t)ch0 * state;
    const float* al = a_log + (size_t)ch0 * state;
    float s_in[N], a_in[N];
#pragma unroll
    for (int j = 0; j < N; ++j) {
        const int i = tid + 256 * j;
        const int ii = i < run ? i : 0;
        s_in[j] = MODE == 1 ? 0.f : src[ii];
        a_in[j] = al[ii];
    }
    const float bias = to_f32(dt_bias[cc]), Dc = skip[cc];
    float dsum = 0.f;
    float xv = x[(size_t)t0 * x_stride + cc], rv = to_f32(raw[(size_t)t0 * raw_stride + cc]);
    float zv = MODE == 1 ? 0.f : to_f32(z[(size_t)t0 * z_stride + cc]);
#pragma unroll
    for (int j = 0; j < N; ++j) {
        const int i = tid + 256 * j;
        if (i < run) stage[(i / state) * (N + 1) + i % state] = s_in[j];
    }
    __syncthreads();
#pragma unroll
    for (int n = 0; n < N; ++n) S[n] = (n < state && active) ? stage[tid * (N + 1) + n] : 0.f;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < N; ++j) {
        const int i = tid + 256 * j;
        if (i < run) stage[(i / state) * (N + 1) + i % state] = a_in[j];
    }
    __syncthreads();
#pragma unroll
    for (int n = 0; n < N; ++n) A2[n] = (n < state && active) ? -expf(stage[tid * (N + 1) + n]) * 1.4426950408889634f : 0.f;
    for (int tile = t0; tile < t1; tile += SC_TT) {
        __syncthreads();                                     // the tile before this one has been read by every thread
        for (int i = tid; i < SC_TT * N; i += 256) {
            const int tt = i / N, n = i % N, t = tile + tt;
            const bool ok = t < t1 && n < state;
            Bs[tt][n] = ok ? to_f32(B[(size_t)t * bc_stride + n]) : 0.f;
            Cs[tt][n] = (ok && MODE != 1) ? to_f32(C[(size_t)t * bc_stride + n]) : 0.f;
        }
        __syncthreads();
        const int count = min(SC_TT, t1 - tile);
        for (int tt = 0; tt < count; ++tt) {
            const int t = tile + tt, tn = t + 1 < t1 ? t + 1 : t;
            const float xn = x[(size_t)tn * x_stride + cc], rn = to_f32(raw[(size_t)tn * raw_stride + cc]);
            const float zn = MODE == 1 ? 0.f : to_f32(z[(size_t)tn * z_stride + cc]);
            const float dt = ss_softplus(rv + bias);
            const float dx = dt * xv;
            dsum += dt;
            float y = 0.f;
#pragma unroll
            for (int n = 0; n < N; ++n) {
                S[n] = fmaf(__builtin_amdgcn_exp2f(dt * A2[n]), S[n], dx * Bs[tt][n]);
                y = fmaf(S[n], Cs[tt][n], y);
            }
            if (MODE != 1 && active) {
                y = fmaf(Dc, xv, y);
                out[(size_t)t * out_stride + c] = from_f32<T>(y * (zv / (1.0f + expf(-zv))));
            }
            xv = xn; rv = rn; zv = zn;
        }
    }
    if (MODE == 2) return;
    __syncthreads();
#pragma unroll
    for (int n = 0; n < N; ++n)
        if (n < state) stage[tid * (N + 1) + n] = S[n];
    __syncthreads();
    float* dst = (MODE == 0 ? pool + (size_t)state_out[sgm] * inner * state : ws_state + slot * inner * state) + (size_t)ch0 * state;
    for (int i = tid; i < run; i += 256) dst[i] = stage[(i / state) * (N + 1) + i % state];
    if (MODE == 1 && active) ws_dt[slot * inner + c] = dsum;
}

// The pieces' start states, piece after piece: a thread a (segment, channel, state entry).  ws_state holds every piece's end
// state from zero and receives its start state; the segment's end state goes to its row of the pool.
__global__ void __launch_bounds__(256)
selective_scan_join_kernel(float* __restrict__ ws_state, const float* __restrict__ ws_dt, const float* __restrict__ a_log,
                           float* __restrict__ pool, const int* __restrict__ state_in, const int* __restrict__ state_out,
                           const int* __restrict__ seg_offsets, int inner, int state, int piece) {
    const int sgm = blockIdx.y;
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= (long)inner * state) return;
    const int c = (int)(i / state);
    const int len = seg_offsets[sgm + 1] - seg_offsets[sgm];
    if (len <= 0) return;
    const int pieces = (len + piece - 1) / piece;
    const size_t base = (size_t)ss_piece_base(seg_offsets, sgm, piece);
    const float A = -expf(a_log[i]);
    float S = pool[(size_t)state_in[sgm] * inner * state + i];
    for (int p = 0; p < pieces; ++p) {
        float* cell = ws_state + (base + p) * inner * state + i;
        const float local = *cell;
        *cell = S;
        S = fmaf(expf(A * ws_dt[(base + p) * inner + c]), S, local);
    }
    pool[(size_t)state_out[sgm] * inner * state + i] = S;
}

extern "C" int ilm_selective_scan_max_state() { return 256; }

// out [T, inner]; x float32 [T, inner]; raw, z [T, inner]; B, C [T, state] (rows of one stride); a_log [inner, state] and
// skip [inner] float32; pool float32 [rows, inner, state]; segment r covers rows seg_offsets[r] .. seg_offsets[r + 1] - 1.
// piece > 0: segments are cut into pieces of that many tokens (max_pieces: the most pieces a segment has; ws_state
// [slots, inner, state] and ws_dt [slots, inner] floats with slots >= the number of pieces of all segments).
extern "C" int ilm_selective_scan(void* out, int out_stride, const void* x, int x_stride, const void* raw, int raw_stride,
                                  const void* dt_bias, const void* B, const void* C, int bc_stride, const void* z, int z_stride,
                                  const void* a_log, const void* skip, void* pool, const void* state_in, const void* state_out,
                                  const void* seg_offsets, int segments, int inner, int state, int piece, int max_pieces, void* ws_state,
                                  void* ws_dt, int dtype, int w_dt, hipStream_t stream) {
    ILM_REQUIRE(segments > 0 && segments <= 65535 && inner > 0 && state > 0, "selective_scan: bad sizes");
    ILM_REQUIRE(state <= ilm_selective_scan_max_state(), "selective_scan: %d state entries a channel (at most %d)", state,
                ilm_selective_scan_max_state());
    ILM_REQUIRE(out_stride >= inner && x_stride >= inner && raw_stride >= inner && z_stride >= inner && bc_stride >= state,
                "selective_scan: rows shorter than their channels");
    ILM_REQUIRE(piece == 0 || (piece > 0 && max_pieces > 0 && max_pieces <= 65535 && ws_state != nullptr && ws_dt != nullptr),
                "selective_scan: pieces need their number and a workspace");
    const int regs = (state + 15) / 16;
    // small states with enough channels to fill blocks of 256: a thread a channel; otherwise a channel's state across 16 lanes
    const bool by_channel = state <= 32 && inner >= 256;
    // decoded tokens and short portions: four channels a lane group where the registers allow, so that a block's loads are in
    // flight together and the launch has a quarter of the blocks
    const int ch = (piece == 0 && regs <= 2 && inner >= 64) ? 4 : 1;
    dim3 grid((inner + 16 * ch - 1) / (16 * ch), segments, piece > 0 ? max_pieces : 1);
#define SS_ARGS(T__, TW__) (T__*)out, out_stride, (const float*)x, x_stride, (const T__*)raw, raw_stride, (const TW__*)dt_bias,       \
                           (const T__*)B, (const T__*)C, bc_stride, (const T__*)z, z_stride, (const float*)a_log, (const float*)skip, \
                           (float*)pool, (const int*)state_in, (const int*)state_out, (const int*)seg_offsets, inner, state, piece,    \
                           (float*)ws_state, (float*)ws_dt
#define SS_MODE(T__, TW__, R__, MODE__)                                                                                 \
    if (ch == 4 && MODE__ == 0 && R__ <= 2) selective_scan_kernel<T__, TW__, (R__ <= 2 ? R__ : 1), 4, 0><<<grid, 256, 0, stream>>>(SS_ARGS(T__, TW__)); \
    else selective_scan_kernel<T__, TW__, R__, 1, MODE__><<<grid, 256, 0, stream>>>(SS_ARGS(T__, TW__));
#define SS_BY_R(T__, TW__, MODE__)                               \
    {                                                            \
        if (regs <= 1) { SS_MODE(T__, TW__, 1, MODE__) }         \
        else if (regs <= 2) { SS_MODE(T__, TW__, 2, MODE__) }    \
        else if (regs <= 4) { SS_MODE(T__, TW__, 4, MODE__) }    \
        else if (regs <= 8) { SS_MODE(T__, TW__, 8, MODE__) }    \
        else { SS_MODE(T__, TW__, 16, MODE__) }                  \
    }
#define SC_BY_N(T__, TW__, MODE__)                                                                                         \
    {                                                                                                                      \
        dim3 cgrid((inner + 255) / 256, segments, piece > 0 ? max_pieces : 1);                                             \
        if (state <= 4) selective_scan_channel_kernel<T__, TW__, 4, MODE__><<<cgrid, 256, 0, stream>>>(SS_ARGS(T__, TW__));       \
        else if (state <= 8) selective_scan_channel_kernel<T__, TW__, 8, MODE__><<<cgrid, 256, 0, stream>>>(SS_ARGS(T__, TW__));  \
        else if (state <= 16) selective_scan_channel_kernel<T__, TW__, 16, MODE__><<<cgrid, 256, 0, stream>>>(SS_ARGS(T__, TW__)); \
        else selective_scan_channel_kernel<T__, TW__, 32, MODE__><<<cgrid, 256, 0, stream>>>(SS_ARGS(T__, TW__));           \
    }
#define SS_BY_DT(MODE__)                                                                                 \
    if (by_channel && dtype == ILM_DTYPE_F32 && w_dt == ILM_DTYPE_F32) SC_BY_N(float, float, MODE__)     \
    else if (by_channel && dtype == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_BF16) SC_BY_N(bf16, bf16, MODE__) \
    else if (by_channel && dtype == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_F32) SC_BY_N(bf16, float, MODE__) \
    else if (dtype == ILM_DTYPE_F32 && w_dt == ILM_DTYPE_F32) SS_BY_R(float, float, MODE__)              \
    else if (dtype == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_BF16) SS_BY_R(bf16, bf16, MODE__)              \
    else if (dtype == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_F32) SS_BY_R(bf16, float, MODE__)              \
    else ILM_REQUIRE(false, "selective_scan: dtypes %d / %d", dtype, w_dt);
    if (piece == 0) {
        SS_BY_DT(0)
        ILM_LAUNCH_CHECK("selective_scan");
        return 0;
    }
    SS_BY_DT(1)
    ILM_LAUNCH_CHECK("selective_scan (pieces from zero)");
    selective_scan_join_kernel<<<dim3((unsigned)(((long)inner * state + 255) / 256), segments), 256, 0, stream>>>(
        (float*)ws_state, (const float*)ws_dt, (const float*)a_log, (float*)pool, (const int*)state_in, (const int*)state_out,
        (const int*)seg_offsets, inner, state, piece);
    ILM_LAUNCH_CHECK("selective_scan (join)");
    SS_BY_DT(2)
    ILM_LAUNCH_CHECK("selective_scan (pieces with outputs)");
#undef SS_BY_DT
#undef SC_BY_N
#undef SS_BY_R
#undef SS_MODE
#undef SS_ARGS
    return 0;
}
