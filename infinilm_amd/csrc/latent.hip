// Attention over a small latent row a token, in its absorbed form: the cache holds, for every token, the normed
// latent c [rank] and one rotated key part [dr] shared by the heads; a query head's unrotated part is carried into
// the latent space (q_h^T W_uk,h, a product per head), so that the scores are plain dot products of rows of
// rank + dr entries against one cached key row, and the values are the latent rows themselves, carried out of the
// latent space after the attention (W_uv,h times the head's result).  The attention itself is the paged kernels'
// with one key/value head of d >= rank + dr entries.
//
//   ilm_latent_prep   from the fused projection rows [q: H (dn + dr) | down: rank + dr] (or, without rotated entries, from
//       rows that hold `down` at any offset: the queries then come from elsewhere): c = RMS norm of the first
//       rank entries of `down` times a weight; the last dr entries and every head's last dr query entries turned
//       in pairs (2i, 2i + 1) by pos * freq[i]; key row [c | turned part | zeros] and value column [c | zeros] into
//       the cache; the turned query parts (and zeros behind them) into the attention's query rows [T, H, d].
//   ilm_head_gemm     out[t, h, n] = sum_k x[t, h, k] W[h, k, n] with strides for every axis (a product per head),
//       float sums in ascending k whatever the number of rows.
#include "common.h"

template <typename T, typename TW>
__global__ void __launch_bounds__(256)
latent_prep_kernel(const T* __restrict__ rows, T* __restrict__ qx, const int* __restrict__ pos, const float* __restrict__ freq,
                   const TW* __restrict__ w, T* __restrict__ kc, T* __restrict__ vc, const int* __restrict__ slots,
                   int H, int dn, int dr, int rank, int d, float eps, int page, int stride, int down_off) {
    extern __shared__ float c[];
    __shared__ float red[4];
    const int t = blockIdx.x, tid = threadIdx.x;
    const T* row = rows + (size_t)t * stride;
    const T* down = row + down_off;
    float ss = 0.f;
    for (int e = tid; e < rank; e += 256) {
        const float v = to_f32(down[e]);
        c[e] = v;
        ss = fmaf(v, v, ss);
    }
    const float rstd = 1.0f / sqrtf(block_sum<4>(ss, red) / (float)rank + eps);
    const float p = (float)pos[t];
    const int slot = slots != nullptr ? slots[t] : -1;
    if (slot >= 0) {
        const int pg = slot / page, off = slot % page;
        T* kdst = kc + ((size_t)pg * page + off) * d;
        T* vdst = vc + (size_t)pg * d * page + off;
        for (int e = tid; e < d; e += 256) {
            float kv = 0.f, vv = 0.f;
            if (e < rank) {
                kv = vv = c[e] * rstd * to_f32(w[e]);
            } else if (e < rank + dr) {
                const int i = (e - rank) >> 1;
                float sn, cs;
                sincosf(p * freq[i], &sn, &cs);
                const float u = to_f32(down[rank + 2 * i]), v = to_f32(down[rank + 2 * i + 1]);
                kv = ((e - rank) & 1) ? v * cs + u * sn : u * cs - v * sn;
            }
            kdst[e] = from_f32<T>(kv);
            vdst[(size_t)e * page] = from_f32<T>(vv);
        }
    }
    // the queries' turned parts and the zeros behind them
    const int tail = d - rank;
    for (int idx = tid; idx < H * tail; idx += 256) {
        const int h = idx / tail, e = idx % tail;
        float y = 0.f;
        if (e < dr) {
            const int i = e >> 1;
            float sn, cs;
            sincosf(p * freq[i], &sn, &cs);
            const T* qr = row + (size_t)h * (dn + dr) + dn;
            const float u = to_f32(qr[2 * i]), v = to_f32(qr[2 * i + 1]);
            y = (e & 1) ? v * cs + u * sn : u * cs - v * sn;
        }
        qx[((size_t)t * H + h) * d + rank + e] = from_f32<T>(y);
    }
}

extern "C" int ilm_latent_prep(const void* rows, void* qx, const void* pos, const void* freq, const void* w, void* kc, void* vc,
                               const void* slots, int T_, int H, int dn, int dr, int rank, int d, float eps, int page,
                               int stride, int down_off, int dtype, int w_dt, hipStream_t stream) {
    if (down_off < 0) down_off = H * (dn + dr);
    ILM_REQUIRE(T_ > 0 && H > 0 && dn > 0 && dr >= 0 && rank > 0 && page > 0, "latent_prep: bad sizes");
    ILM_REQUIRE(dr % 2 == 0 && d >= rank + dr && rank <= 8192, "latent_prep: %d + %d entries in rows of %d", rank, dr, d);
    ILM_REQUIRE(stride >= down_off + rank + dr && (dr == 0 || stride >= H * (dn + dr)), "latent_prep: rows of %d do not hold the projections", stride);
    ILM_REQUIRE(dr == 0 || freq != nullptr, "latent_prep: a rotation needs frequencies");
    const size_t shm = (size_t)rank * sizeof(float);
#define LP_LAUNCH(T__, TW__)                                                                                          \
    latent_prep_kernel<T__, TW__><<<T_, 256, shm, stream>>>((const T__*)rows, (T__*)qx, (const int*)pos, (const float*)freq, \
                                                            (const TW__*)w, (T__*)kc, (T__*)vc, (const int*)slots, H, dn, dr, \
                                                            rank, d, eps, page, stride, down_off)
    if (dtype == ILM_DTYPE_F32 && w_dt == ILM_DTYPE_F32) LP_LAUNCH(float, float);
    else if (dtype == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_BF16) LP_LAUNCH(bf16, bf16);
    else if (dtype == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_F32) LP_LAUNCH(bf16, float);
    else ILM_REQUIRE(false, "latent_prep: dtypes %d / %d", dtype, w_dt);
#undef LP_LAUNCH
    ILM_LAUNCH_CHECK("latent_prep");
    return 0;
}

// ------------------------------------------------------------------------------------------
// A product per head.  A block: 16 rows x 64 outputs of one head; x and W pass through LDS in steps of 64 k.
// Thread (n, row group) holds 4 rows of one output column.  W's fast axis may be k or n; the tile is loaded along it.
// ------------------------------------------------------------------------------------------
#define HG_ROWS 16
#define HG_COLS 64
#define HG_K 64

template <typename T, typename TO>
__global__ void __launch_bounds__(256)
head_gemm_kernel(TO* __restrict__ out, const T* __restrict__ x, const T* __restrict__ w, int M, int N, int K, long x_t, long x_h,
                 long w_h, long w_k, long w_n, long o_t, long o_h) {
    __shared__ float xs[HG_ROWS][HG_K + 1];
    __shared__ float ws[HG_K][HG_COLS + 1];
    const int h = blockIdx.z, n0 = blockIdx.x * HG_COLS, m0 = blockIdx.y * HG_ROWS, tid = threadIdx.x;
    const int nl = tid & 63, rg = tid >> 6;
    const T* xh = x + (size_t)h * x_h;
    const T* wh = w + (size_t)h * w_h;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < K; k0 += HG_K) {
        for (int i = tid; i < HG_ROWS * HG_K; i += 256) {
            const int r = i / HG_K, kk = i % HG_K;
            xs[r][kk] = (m0 + r < M && k0 + kk < K) ? to_f32(xh[(size_t)(m0 + r) * x_t + k0 + kk]) : 0.f;
        }
        for (int i = tid; i < HG_K * HG_COLS; i += 256) {
            const int kk = w_n == 1 ? i / HG_COLS : i % HG_K, nn = w_n == 1 ? i % HG_COLS : i / HG_K;
            ws[kk][nn] = (k0 + kk < K && n0 + nn < N) ? to_f32(wh[(size_t)(k0 + kk) * w_k + (size_t)(n0 + nn) * w_n]) : 0.f;
        }
        __syncthreads();
#pragma unroll 8
        for (int kk = 0; kk < HG_K; ++kk) {
            const float wv = ws[kk][nl];
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[r] = fmaf(xs[rg * 4 + r][kk], wv, acc[r]);
        }
        __syncthreads();
    }
    if (n0 + nl < N)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int m = m0 + rg * 4 + r;
            if (m < M) out[(size_t)m * o_t + (size_t)h * o_h + n0 + nl] = from_f32<TO>(acc[r]);
        }
}

// The same for few rows of bfloat16 on the matrix cores: a wave owns one head and 16 outputs for up to 64 rows (four row tiles
// that share every fragment of W), k in steps of 32 with all of a step's loads independent of each other; nothing passes LDS.
// x rows, K and the strides of x in multiples of 8 elements (16-byte loads); W with k dense (16-byte loads) or n dense (eight
// 2-byte loads a fragment).  A row's sum is its own: rows beyond T are zeros and are not stored.
typedef __attribute__((ext_vector_type(8))) __bf16 hg_bf16x8;
typedef __attribute__((ext_vector_type(4))) float hg_f32x4;

template <bool W_K_DENSE>
__global__ void __launch_bounds__(256)
head_gemm_mfma_kernel(bf16* __restrict__ out, const bf16* __restrict__ x, const bf16* __restrict__ w, int M, int N, int K, int H,
                      long x_t, long x_h, long w_h, long w_k, long w_n, long o_t, long o_h) {
    const int n_tiles = (N + 15) >> 4;
    const int item = blockIdx.x * 4 + (threadIdx.x >> 6);          // (head, tile of 16 outputs)
    if (item >= H * n_tiles) return;
    const int h = item / n_tiles, n0 = (item % n_tiles) * 16, m0 = blockIdx.y * 64;
    const int lane = threadIdx.x & 63, r16 = lane & 15, q = lane >> 4;
    const bf16* xh = x + (size_t)h * x_h;
    const bf16* wh = w + (size_t)h * w_h;
    const int n = n0 + r16;
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    hg_f32x4 acc[4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) acc[rt] = hg_f32x4{0.f, 0.f, 0.f, 0.f};
    const int row_tiles = (M - m0 + 15) >> 4 < 4 ? (M - m0 + 15) >> 4 : 4;
#pragma unroll 2
    for (int k0 = 0; k0 < K; k0 += 32) {
        const int k = k0 + q * 8;
        uint4 b = zero;
        if (k < K && n < N) {
            if (W_K_DENSE) {
                b = *reinterpret_cast<const uint4*>(wh + (size_t)n * w_n + k);
            } else {
                uint32_t e[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) e[j] = (wh + (size_t)(k + j) * w_k)[n].bits;
                b = make_uint4(e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16));
            }
        }
        uint4 a[4];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
            const int m = m0 + rt * 16 + r16;
            a[rt] = (rt < row_tiles && m < M && k < K) ? *reinterpret_cast<const uint4*>(xh + (size_t)m * x_t + k) : zero;
        }
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
            if (rt < row_tiles)
                acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(hg_bf16x8, a[rt]), __builtin_bit_cast(hg_bf16x8, b),
                                                                  acc[rt], 0, 0, 0);
    }
    // lane holds rows m0 + 16 rt + 4 q + i and output n
    if (n < N)
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int m = m0 + rt * 16 + q * 4 + i;
                if (rt < row_tiles && m < M) out[(size_t)m * o_t + (size_t)h * o_h + n] = from_f32<bf16>(acc[rt][i]);
            }
}

extern "C" int ilm_head_gemm_mfma(void* out, const void* x, const void* w, int M, int N, int K, int H, long x_t, long x_h, long w_h,
                                  long w_k, long w_n, long o_t, long o_h, hipStream_t stream) {
    ILM_REQUIRE(M > 0 && N > 0 && K > 0 && H > 0, "head_gemm_mfma: bad sizes");
    ILM_REQUIRE(K % 8 == 0 && x_t % 8 == 0 && x_h % 8 == 0 && ((uintptr_t)x % 16) == 0, "head_gemm_mfma: rows of x must allow 16-byte loads");
    ILM_REQUIRE(w_k == 1 || w_n == 1, "head_gemm_mfma: one axis of W must be dense");
    ILM_REQUIRE(w_k != 1 || (w_n % 8 == 0 && w_h % 8 == 0 && ((uintptr_t)w % 16) == 0), "head_gemm_mfma: rows of W must allow 16-byte loads");
    const long items = (long)H * ((N + 15) / 16);
    ILM_REQUIRE(items < (1L << 30) && (M + 63) / 64 <= 65535, "head_gemm_mfma: too large");
    dim3 grid((unsigned)((items + 3) / 4), (M + 63) / 64);
    if (w_k == 1)
        head_gemm_mfma_kernel<true><<<grid, 256, 0, stream>>>((bf16*)out, (const bf16*)x, (const bf16*)w, M, N, K, H, x_t, x_h, w_h, w_k, w_n, o_t, o_h);
    else
        head_gemm_mfma_kernel<false><<<grid, 256, 0, stream>>>((bf16*)out, (const bf16*)x, (const bf16*)w, M, N, K, H, x_t, x_h, w_h, w_k, w_n, o_t, o_h);
    ILM_LAUNCH_CHECK("head_gemm_mfma");
    return 0;
}

extern "C" int ilm_head_gemm(void* out, const void* x, const void* w, int M, int N, int K, int H, long x_t, long x_h, long w_h,
                             long w_k, long w_n, long o_t, long o_h, int dtype, int out_dt, hipStream_t stream) {
    ILM_REQUIRE(M > 0 && N > 0 && K > 0 && H > 0 && H <= 65535, "head_gemm: bad sizes");
    ILM_REQUIRE((M + HG_ROWS - 1) / HG_ROWS <= 65535, "head_gemm: too many rows");
    ILM_REQUIRE(w_k == 1 || w_n == 1, "head_gemm: one axis of W must be dense");
    dim3 grid((N + HG_COLS - 1) / HG_COLS, (M + HG_ROWS - 1) / HG_ROWS, H);
#define HG_LAUNCH(T__, TO__)                                                                                              \
    head_gemm_kernel<T__, TO__><<<grid, 256, 0, stream>>>((TO__*)out, (const T__*)x, (const T__*)w, M, N, K, x_t, x_h, w_h, \
                                                          w_k, w_n, o_t, o_h)
    if (dtype == ILM_DTYPE_F32 && out_dt == ILM_DTYPE_F32) HG_LAUNCH(float, float);
    else if (dtype == ILM_DTYPE_BF16 && out_dt == ILM_DTYPE_BF16) HG_LAUNCH(bf16, bf16);
    else if (dtype == ILM_DTYPE_BF16 && out_dt == ILM_DTYPE_F32) HG_LAUNCH(bf16, float);
    else ILM_REQUIRE(false, "head_gemm: dtypes %d / %d", dtype, out_dt);
#undef HG_LAUNCH
    ILM_LAUNCH_CHECK("head_gemm");
    return 0;
}
