// Attention whose scores are mixed over the heads before the softmax, with a learned term in the denominator,
// and the step that makes its queries, keys and values ready.
//
//   ilm_qkv_norm_rope_kvwrite   per head of the fused projection rows [T, (nh + 2 nkv) d]: an RMS norm over the first
//       dn entries of every q and k head with a weight shared by the heads (or none), a turn of the entry pairs
//       (2i, 2i + 1), i < rd / 2, by the angle pos * freq[i], every value head divided by its root mean square
//       over its first dv entries (or not); q and k are rewritten in place, k and v go to the paged cache.
//   ilm_attn_headmix            raw_g(j) = scale q_g . k_kv(g),j;  s_h(j) = sum_g M[h, g] raw_g(j);  over the keys j
//       the token sees (its last `window` positions and the sequence's first `keep_first`, or all): p_h(j) = exp(s_h(j)) / (sum_j' exp(s_h(j')) + exp(sink_h));
//       o_h = sum_j p_h(j) v_kv(h),j.  M and sink may be absent (identity, no term).
//
// All arithmetic is float.  The attention is the plain form: one block a token walks the keys in tiles of 64 aligned
// to the absolute key index and keeps a running maximum, sum and output per head, so a token's result is a function
// of its position and its request's cache alone: cutting a prompt or batching it changes no bit.
#include "common.h"

__device__ __forceinline__ void hm_load4(const float* p, float* v) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void hm_load4(const bf16* p, float* v) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
    v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
}

// ------------------------------------------------------------------------------------------
// One wave a (token, head); the head's d entries pass through LDS as floats.
// ------------------------------------------------------------------------------------------
template <typename T, typename TW>
__global__ void __launch_bounds__(256)
qkv_norm_rope_kvwrite_kernel(T* __restrict__ qkv, const int* __restrict__ pos, const float* __restrict__ freq,
                             const TW* __restrict__ wq, const TW* __restrict__ wk, T* __restrict__ kc, T* __restrict__ vc,
                             const int* __restrict__ slots, int nh, int nkv, int d, int dn, int dv, int rd, int v_norm,
                             float eps, int page, int stride) {
    extern __shared__ float smem[];
    const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int head = blockIdx.y * 4 + wave;
    const bool active = head < nh + 2 * nkv;      // (waves beyond the last head go along to the barriers and do nothing)
    float* x = smem + wave * d;
    T* src = qkv + (size_t)t * stride + (size_t)(active ? head : 0) * d;
    const bool is_q = head < nh, is_k = !is_q && head < nh + nkv;
    const int n = (is_q || is_k) ? dn : dv;       // the entries that count
    float ss = 0.f;
    if (active)
        for (int e = lane; e < d; e += 64) {
            const float v = e < n ? to_f32(src[e]) : 0.f;
            x[e] = v;
            ss = fmaf(v, v, ss);
        }
    ss = wave_sum(ss);
    const TW* w = is_q ? wq : (is_k ? wk : nullptr);
    const bool normed = (is_q || is_k) ? (w != nullptr) : (v_norm != 0);
    const float rstd = normed ? 1.0f / sqrtf(ss / (float)n + eps) : 1.0f;
    if (active)
        for (int e = lane; e < n; e += 64) x[e] = x[e] * rstd * ((w != nullptr) ? to_f32(w[e]) : 1.0f);
    __syncthreads();
    if (active && (is_q || is_k) && rd > 0) {
        const float p = (float)pos[t];
        for (int i = lane; i < rd / 2; i += 64) {
            float sn, cs;
            sincosf(p * freq[i], &sn, &cs);
            const float u = x[2 * i], v = x[2 * i + 1];
            x[2 * i] = u * cs - v * sn;
            x[2 * i + 1] = v * cs + u * sn;
        }
    }
    __syncthreads();
    if (!active) return;
    const int slot = (slots != nullptr && !is_q) ? slots[t] : -1;
    if (is_q || is_k)
        for (int e = lane; e < d; e += 64) src[e] = from_f32<T>(x[e]);
    if (slot >= 0) {
        const int pg = slot / page, off = slot % page;
        if (is_k) {
            T* dst = kc + (((size_t)pg * nkv + (head - nh)) * page + off) * d;
            for (int e = lane; e < d; e += 64) dst[e] = from_f32<T>(x[e]);
        } else {
            T* dst = vc + ((size_t)pg * nkv + (head - nh - nkv)) * d * page + off;
            for (int e = lane; e < d; e += 64) dst[(size_t)e * page] = from_f32<T>(x[e]);
        }
    }
}

extern "C" int ilm_qkv_norm_rope_kvwrite(void* qkv, const void* pos, const void* freq, const void* wq, const void* wk,
                                         void* kc, void* vc, const void* slots, int T_, int nh, int nkv, int d, int dn, int dv,
                                         int rd, int v_norm, float eps, int page, int stride, int dtype, int w_dt,
                                         hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && nh > 0 && nkv > 0 && d > 0 && page > 0, "qkv_norm_rope_kvwrite: bad sizes");
    ILM_REQUIRE(dn > 0 && dn <= d && dv > 0 && dv <= d, "qkv_norm_rope_kvwrite: %d / %d entries that count in heads of %d", dn, dv, d);
    ILM_REQUIRE(rd >= 0 && rd % 2 == 0 && rd <= dn && (rd == 0 || freq != nullptr), "qkv_norm_rope_kvwrite: %d turned entries", rd);
    ILM_REQUIRE((wq == nullptr) == (wk == nullptr), "qkv_norm_rope_kvwrite: a norm weight for q and k, or for neither");
    ILM_REQUIRE(d <= 4096 && T_ <= 0x7fffffff / 1, "qkv_norm_rope_kvwrite: head size %d", d);
    ILM_REQUIRE(slots == nullptr || (kc != nullptr && vc != nullptr), "qkv_norm_rope_kvwrite: slots without a cache");
    dim3 grid(T_, (nh + 2 * nkv + 3) / 4);
    const size_t shm = (size_t)4 * d * sizeof(float);
#define QN_LAUNCH(T__, TW__)                                                                                              \
    qkv_norm_rope_kvwrite_kernel<T__, TW__><<<grid, 256, shm, stream>>>(                                                  \
        (T__*)qkv, (const int*)pos, (const float*)freq, (const TW__*)wq, (const TW__*)wk, (T__*)kc, (T__*)vc,              \
        (const int*)slots, nh, nkv, d, dn, dv, rd, v_norm, eps, page, stride)
    if (dtype == ILM_DTYPE_F32 && w_dt == ILM_DTYPE_F32) QN_LAUNCH(float, float);
    else if (dtype == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_BF16) QN_LAUNCH(bf16, bf16);
    else if (dtype == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_F32) QN_LAUNCH(bf16, float);
    else ILM_REQUIRE(false, "qkv_norm_rope_kvwrite: dtypes %d / %d", dtype, w_dt);
#undef QN_LAUNCH
    ILM_LAUNCH_CHECK("qkv_norm_rope_kvwrite");
    return 0;
}

// ------------------------------------------------------------------------------------------
// The attention.  LDS (floats): q [nh d] | raw scores [nh 64] | weights [nh 64] | M [nh nh] | running max, sum,
// correction [3 nh] | outputs [nh dv].
// ------------------------------------------------------------------------------------------
#define HM_R 8     // heads of one group whose scores a lane forms from one read of the key

template <typename T, bool VEC>
__global__ void __launch_bounds__(256)
attn_headmix_kernel(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ kc, const T* __restrict__ vc,
                    const int* __restrict__ block_tables, const int* __restrict__ seg, const int* __restrict__ pos,
                    const int* __restrict__ rows, const float* __restrict__ mix, const float* __restrict__ sink,
                    int nh, int nkv, int d, int dv, int page, int max_blocks, int q_stride, int out_stride, float scale,
                    int window, int keep_first) {
    extern __shared__ float smem[];
    float* qs = smem;
    float* raw = qs + nh * d;
    float* wt = raw + nh * 64;
    float* mx = wt + nh * 64;
    float* run_m = mx + nh * nh;
    float* run_l = run_m + nh;
    float* corr = run_l + nh;
    float* acc = corr + nh;
    const int t = rows != nullptr ? rows[blockIdx.x] : (int)blockIdx.x;
    if (t < 0) return;                               // an entry of the row list that names no row
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int p = pos[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int keep = lo < keep_first ? lo : keep_first;     // the first tokens stay seen below the window's edge: keys 0 .. keep - 1
    const int* bt = block_tables + (size_t)seg[t] * max_blocks;
    const T* qrow = q + (size_t)t * q_stride;
    const int per = nh / nkv;
    for (int i = tid; i < nh * d; i += 256) qs[i] = to_f32(qrow[i]);
    for (int i = tid; i < nh * nh; i += 256) mx[i] = mix != nullptr ? mix[i] : ((i / nh == i % nh) ? 1.f : 0.f);
    for (int i = tid; i < nh; i += 256) { run_m[i] = -INFINITY; run_l[i] = 0.f; }
    for (int i = tid; i < nh * dv; i += 256) acc[i] = 0.f;
    __syncthreads();
    const int chunks = (per + HM_R - 1) / HM_R;      // pieces of a group of at most HM_R heads
    for (int tile = keep > 0 ? 0 : lo >> 6; tile <= (p >> 6); ++tile) {
        if ((tile << 6) + 63 < lo && (tile << 6) >= keep) continue;       // between the kept keys and the window
        const int key = (tile << 6) + lane;
        const bool valid = key <= p && (key >= lo || key < keep);
        // 1. raw scores of all heads for the tile's keys: a wave takes (group, piece) items in turn, a lane a key
        for (int item = wave; item < nkv * chunks; item += 4) {
            const int c = item / chunks, g0 = c * per + (item % chunks) * HM_R;
            const int gn = min(HM_R, (c + 1) * per - g0);
            float dot[HM_R];
#pragma unroll
            for (int r = 0; r < HM_R; ++r) dot[r] = 0.f;
            if (valid) {
                const int pg = bt[key / page];
                const T* krow = kc + (((size_t)pg * nkv + c) * page + (key % page)) * d;
                if (VEC) {
                    for (int i = 0; i < d; i += 4) {
                        float kv[4];
                        hm_load4(krow + i, kv);
#pragma unroll
                        for (int r = 0; r < HM_R; ++r) {
                            if (r < gn) {
                                const float* qq = qs + (g0 + r) * d + i;
#pragma unroll
                                for (int e = 0; e < 4; ++e) dot[r] = fmaf(qq[e], kv[e], dot[r]);
                            }
                        }
                    }
                } else {
                    for (int i = 0; i < d; ++i) {
                        const float kv = to_f32(krow[i]);
#pragma unroll
                        for (int r = 0; r < HM_R; ++r)
                            if (r < gn) dot[r] = fmaf(qs[(g0 + r) * d + i], kv, dot[r]);
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < HM_R; ++r)
                if (r < gn) raw[(g0 + r) * 64 + lane] = dot[r] * scale;
        }
        __syncthreads();
        // 2. mixed scores, running maximum and sum, the tile's weights: a wave takes heads in turn
        for (int h = wave; h < nh; h += 4) {
            float s = 0.f;
            for (int g = 0; g < nh; ++g) s = fmaf(mx[h * nh + g], raw[g * 64 + lane], s);
            if (!valid) s = -INFINITY;
            const float m_old = run_m[h];
            const float m_new = fmaxf(m_old, wave_max(s));
            const float pj = valid ? expf(s - m_new) : 0.f;
            const float cf = expf(m_old - m_new);
            const float l_new = run_l[h] * cf + wave_sum(pj);
            wt[h * 64 + lane] = pj;
            if (lane == 0) { run_m[h] = m_new; run_l[h] = l_new; corr[h] = cf; }
        }
        __syncthreads();
        // 3. outputs: a thread takes (head, value entry) items in turn and walks the tile's seen keys in ascending order: the
        //    kept first keys, then the window's
        for (int idx = tid; idx < nh * dv; idx += 256) {
            const int h = idx / dv, e = idx % dv, c = h / per;
            float a = acc[idx] * corr[h];
            const float* wrow = wt + h * 64;
            for (int part = keep > (tile << 6) ? 0 : 1; part < 2; ++part) {
                const int j0 = part == 0 ? 0 : (lo > (tile << 6) ? lo - (tile << 6) : 0);
                const int j1 = part == 0 ? min(63, keep - 1 - (tile << 6)) : ((p - (tile << 6)) < 63 ? p - (tile << 6) : 63);
                int j = j0;
                if (VEC) {
                    for (; j <= j1 && (j & 3); ++j) {
                        const int kk = (tile << 6) + j;
                        a = fmaf(wrow[j], to_f32(vc[(((size_t)bt[kk / page] * nkv + c) * d + e) * page + (kk % page)]), a);
                    }
                    for (; j + 3 <= j1; j += 4) {
                        const int kk = (tile << 6) + j;
                        float vv[4];
                        hm_load4(vc + (((size_t)bt[kk / page] * nkv + c) * d + e) * page + (kk % page), vv);
                        a = fmaf(wrow[j], vv[0], a);
                        a = fmaf(wrow[j + 1], vv[1], a);
                        a = fmaf(wrow[j + 2], vv[2], a);
                        a = fmaf(wrow[j + 3], vv[3], a);
                    }
                }
                for (; j <= j1; ++j) {
                    const int kk = (tile << 6) + j;
                    a = fmaf(wrow[j], to_f32(vc[(((size_t)bt[kk / page] * nkv + c) * d + e) * page + (kk % page)]), a);
                }
            }
            acc[idx] = a;
        }
        __syncthreads();
    }
    T* orow = out + (size_t)t * out_stride;
    for (int idx = tid; idx < nh * d; idx += 256) {
        const int h = idx / d, e = idx % d;
        float y = 0.f;
        if (e < dv) {
            float L = run_l[h];
            if (sink != nullptr) L += expf(sink[h] - run_m[h]);
            y = acc[h * dv + e] / L;
        }
        orow[idx] = from_f32<T>(y);
    }
}

extern "C" long ilm_attn_headmix_lds_bytes(int nh, int d, int dv) {
    return (long)sizeof(float) * ((long)nh * d + 2L * nh * 64 + (long)nh * nh + 3L * nh + (long)nh * dv);
}

// rows: null (every token of the step) or a list of n_rows row numbers (-1: no row)
extern "C" int ilm_attn_headmix(void* out, const void* q, const void* kc, const void* vc, const void* block_tables,
                                const void* seg, const void* pos, const void* rows, int n_rows, const void* mix,
                                const void* sink, int nh, int nkv, int d, int dv, int page, int max_blocks, int q_stride,
                                int out_stride, float scale, int window, int keep_first, int dtype, hipStream_t stream) {
    ILM_REQUIRE(keep_first >= 0, "attn_headmix: %d kept first tokens", keep_first);
    ILM_REQUIRE(n_rows > 0 && nh > 0 && nkv > 0 && d > 0 && page > 0 && max_blocks > 0, "attn_headmix: bad sizes");
    ILM_REQUIRE(nh % nkv == 0, "attn_headmix: %d query heads do not divide into %d groups", nh, nkv);
    ILM_REQUIRE(dv > 0 && dv <= d, "attn_headmix: value size %d in heads of %d", dv, d);
    ILM_REQUIRE(dtype == ILM_DTYPE_F32 || dtype == ILM_DTYPE_BF16, "attn_headmix: unknown dtype %d", dtype);
    const long shm = ilm_attn_headmix_lds_bytes(nh, d, dv);
    ILM_REQUIRE(shm <= 160 * 1024 - 1024, "attn_headmix: %d heads of %d need %ld bytes of LDS, more than a compute unit has", nh, d, shm);
    const bool vec = d % 4 == 0 && page % 4 == 0 && ((uintptr_t)kc & 15) == 0 && ((uintptr_t)vc & 15) == 0;
#define HM_LAUNCH(T_, VEC_)                                                                                              \
    {                                                                                                                    \
        auto kern = attn_headmix_kernel<T_, VEC_>;                                                                       \
        if (shm > 48 * 1024) {                                                                                           \
            hipError_t e_ = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm); \
            ILM_REQUIRE(e_ == hipSuccess, "attn_headmix: %ld bytes of LDS refused: %s", shm, hipGetErrorString(e_));      \
        }                                                                                                                \
        kern<<<n_rows, 256, shm, stream>>>((T_*)out, (const T_*)q, (const T_*)kc, (const T_*)vc, (const int*)block_tables, \
                                           (const int*)seg, (const int*)pos, (const int*)rows, (const float*)mix,        \
                                           (const float*)sink, nh, nkv, d, dv, page, max_blocks, q_stride, out_stride,   \
                                           scale, window, keep_first);                                                   \
    }
    if (dtype == ILM_DTYPE_F32) {
        if (vec) HM_LAUNCH(float, true) else HM_LAUNCH(float, false)
    } else {
        if (vec) HM_LAUNCH(bf16, true) else HM_LAUNCH(bf16, false)
    }
#undef HM_LAUNCH
    ILM_LAUNCH_CHECK("attn_headmix");
    return 0;
}
