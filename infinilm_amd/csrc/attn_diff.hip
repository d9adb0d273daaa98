// Attention whose heads come in several maps over the same values ("differential" attention), and the step that makes
// its queries, keys and values ready.
//
//   ilm_maps_norm_rope_kvwrite   rows [q: H maps dim | k: G maps dim | v: G vdim] (float32 or the activations' dtype, at given
//       offsets of wider rows; k and v may be absent for a layer that reads another layer's cache): every q and k unit of
//       dim entries is RMS-normed with a weight shared by all units (or none) and its first rd entries are turned in the
//       pairs (i, i + rd/2) by the angle pos * freq[i]; q goes to dense rows [T, H maps dim], k to the paged cache with a
//       key/value head's maps side by side ([pages, G, page, d], entry m dim + e), v to the transposed value cache.
//       `spread`: the queries go out as rows of G x d entries a unit instead (zeros but for the unit's own group and map),
//       which is how the matrix-core attention that asks all groups at once takes them.
//   ilm_maps_combine             from float rows [T, H 2, d] of the two maps' results: o = a_0 - lambda a_1, its root mean
//       square over the head's vdim entries, the scale (the end of ilm_attn_maps, for results that another kernel made).
//   ilm_attn_maps                per query head h (key/value head h / (H/G)) and map m a softmax attention of its own over
//       the keys the token sees (j <= i and (i - j < window or j < keep_first); window 0: all), scores scale q_hm . k_gm,
//       optionally one more term exp(sink) in every denominator; the maps' results a_m share the values.  One map: o = a_0.
//       Two maps: o = a_0 - lambda a_1 with lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff, then o / sqrt(mean(o^2) + eps)
//       over the head's vdim entries, times out_scale.
//
// All arithmetic is float.  One block a token walks the keys in tiles of 64 aligned to the absolute key index and keeps a
// running maximum, sum and output per (head, map), so a token's result is a function of its position and its request's
// cache alone: cutting a prompt or batching it changes no bit.
#include "common.h"

template <typename TS, typename T, typename TW>
__global__ void __launch_bounds__(256)
maps_norm_rope_kvwrite_kernel(T* __restrict__ q_out, const TS* __restrict__ src, int stride, int q_off, int k_off, int v_off,
                              const int* __restrict__ pos, const float* __restrict__ freq, const TW* __restrict__ wq,
                              const TW* __restrict__ wk, T* __restrict__ kc, T* __restrict__ vc, const int* __restrict__ slots,
                              int H, int G, int maps, int dim, int vdim, int d, int rd, float eps, int page, int spread) {
    extern __shared__ float smem[];
    const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nq = H * maps, nk = k_off >= 0 ? G * maps : 0, nv = k_off >= 0 ? G : 0;
    const int unit = blockIdx.y * 4 + wave;
    const bool active = unit < nq + nk + nv;
    const bool is_q = unit < nq, is_k = !is_q && unit < nq + nk;
    const int n = (is_q || is_k) ? dim : vdim;
    const int width = dim > vdim ? dim : vdim;
    float* x = smem + wave * width;
    const TS* row = src + (size_t)t * stride;
    const TS* p = is_q ? row + q_off + (size_t)unit * dim
                       : (is_k ? row + k_off + (size_t)(unit - nq) * dim : row + v_off + (size_t)(active ? unit - nq - nk : 0) * vdim);
    float ss = 0.f;
    if (active)
        for (int e = lane; e < n; e += 64) {
            const float v = to_f32(p[e]);
            x[e] = v;
            ss = fmaf(v, v, ss);
        }
    ss = wave_sum(ss);
    const TW* w = is_q ? wq : (is_k ? wk : nullptr);
    if (active && w != nullptr) {
        const float rstd = 1.0f / sqrtf(ss / (float)n + eps);
        for (int e = lane; e < n; e += 64) x[e] = x[e] * rstd * to_f32(w[e]);
    }
    __syncthreads();
    const int half = rd / 2;
    if (active && (is_q || is_k) && rd > 0) {
        const float ps = (float)pos[t];
        for (int i = lane; i < half; i += 64) {      // (a pair a lane and round; no pair is touched by two lanes)
            float sn, cs;
            sincosf(ps * freq[i], &sn, &cs);
            const float u = x[i], v = x[i + half];
            x[i] = u * cs - v * sn;
            x[i + half] = v * cs + u * sn;
        }
    }
    __syncthreads();
    if (!active) return;
    if (is_q && spread) {
        // for the matrix-core kernel that asks every key/value group with one query of G x d entries: unit (h, m) is zeros
        // but for its own group's entries m dim .. (m + 1) dim - 1, so that its score is q_hm . k_gm and nothing else
        const int g = (unit / maps) / (H / G), m = unit % maps;
        T* dst = q_out + ((size_t)t * nq + unit) * G * d;
        for (int e = lane; e < G * d; e += 64) {
            const int c = e / d, i = e % d - m * dim;
            dst[e] = from_f32<T>((c == g && i >= 0 && i < dim) ? x[i] : 0.f);
        }
        return;
    }
    if (is_q) {
        T* dst = q_out + (size_t)t * nq * dim + (size_t)unit * dim;
        for (int e = lane; e < dim; e += 64) dst[e] = from_f32<T>(x[e]);
        return;
    }
    const int slot = slots != nullptr ? slots[t] : -1;
    if (slot < 0) return;
    const int pg = slot / page, off = slot % page;
    if (is_k) {
        const int u = unit - nq, g = u / maps, m = u % maps;
        T* dst = kc + (((size_t)pg * G + g) * page + off) * d + (size_t)m * dim;
        for (int e = lane; e < dim; e += 64) dst[e] = from_f32<T>(x[e]);
    } else {
        const int g = unit - nq - nk;
        T* dst = vc + ((size_t)pg * G + g) * d * page + off;
        for (int e = lane; e < vdim; e += 64) dst[(size_t)e * page] = from_f32<T>(x[e]);
    }
}

extern "C" int ilm_maps_norm_rope_kvwrite(void* q_out, const void* src, int stride, int q_off, int k_off, int v_off, const void* pos,
                                          const void* freq, const void* wq, const void* wk, void* kc, void* vc, const void* slots,
                                          int T_, int H, int G, int maps, int dim, int vdim, int d, int rd, float eps, int page,
                                          int src_dt, int dtype, int w_dt, int spread, hipStream_t stream) {
    ILM_REQUIRE(!spread || (H % G == 0 && maps * dim <= d), "maps_norm_rope_kvwrite: queries spread over %d groups of %d", G, d);
    ILM_REQUIRE(T_ > 0 && H > 0 && G > 0 && maps > 0 && dim > 0 && vdim > 0 && page > 0, "maps_norm_rope_kvwrite: bad sizes");
    ILM_REQUIRE(k_off < 0 || (maps * dim <= d && vdim <= d), "maps_norm_rope_kvwrite: %d maps of %d / values of %d in cache heads of %d", maps,
                dim, vdim, d);
    ILM_REQUIRE(rd >= 0 && rd % 2 == 0 && rd <= dim && (rd == 0 || freq != nullptr), "maps_norm_rope_kvwrite: %d turned entries", rd);
    ILM_REQUIRE(dim <= 4096 && vdim <= 4096, "maps_norm_rope_kvwrite: head sizes %d / %d", dim, vdim);
    ILM_REQUIRE(k_off < 0 || slots == nullptr || (kc != nullptr && vc != nullptr), "maps_norm_rope_kvwrite: slots without a cache");
    const int units = H * maps + (k_off >= 0 ? G * maps + G : 0);
    dim3 grid(T_, (units + 3) / 4);
    const size_t shm = (size_t)4 * (dim > vdim ? dim : vdim) * sizeof(float);
#define MP_LAUNCH(TS__, T__, TW__)                                                                                           \
    maps_norm_rope_kvwrite_kernel<TS__, T__, TW__><<<grid, 256, shm, stream>>>(                                              \
        (T__*)q_out, (const TS__*)src, stride, q_off, k_off, v_off, (const int*)pos, (const float*)freq, (const TW__*)wq,    \
        (const TW__*)wk, (T__*)kc, (T__*)vc, (const int*)slots, H, G, maps, dim, vdim, d, rd, eps, page, spread)
    if (src_dt == ILM_DTYPE_F32 && dtype == ILM_DTYPE_F32 && w_dt == ILM_DTYPE_F32) MP_LAUNCH(float, float, float);
    else if (src_dt == ILM_DTYPE_F32 && dtype == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_BF16) MP_LAUNCH(float, bf16, bf16);
    else if (src_dt == ILM_DTYPE_F32 && dtype == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_F32) MP_LAUNCH(float, bf16, float);
    else if (src_dt == ILM_DTYPE_BF16 && dtype == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_BF16) MP_LAUNCH(bf16, bf16, bf16);
    else if (src_dt == ILM_DTYPE_BF16 && dtype == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_F32) MP_LAUNCH(bf16, bf16, float);
    else ILM_REQUIRE(false, "maps_norm_rope_kvwrite: dtypes %d / %d / %d", src_dt, dtype, w_dt);
#undef MP_LAUNCH
    ILM_LAUNCH_CHECK("maps_norm_rope_kvwrite");
    return 0;
}

// ------------------------------------------------------------------------------------------
// The attention.  LDS (floats): q [VH dim] | raw scores [VH 64] | weights [VH 64] | running max, sum, correction [3 VH] |
// outputs [VH vdim] | lambda; VH = H maps (head h, map m at h maps + m).
// ------------------------------------------------------------------------------------------
#define AM_R 8     // heads of one group and map whose scores a lane forms from one read of the key

template <typename T, typename TW>
__global__ void __launch_bounds__(256)
attn_maps_kernel(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ kc, const T* __restrict__ vc,
                 const int* __restrict__ block_tables, const int* __restrict__ seg, const int* __restrict__ pos,
                 const int* __restrict__ rows, int H, int G, int maps, int dim, int vdim, int d, int page, int max_blocks,
                 int out_stride, float scale, int window, int keep_first, const float* __restrict__ sink,
                 const TW* __restrict__ lq1, const TW* __restrict__ lk1, const TW* __restrict__ lq2, const TW* __restrict__ lk2,
                 float diff, float norm_eps, float out_scale) {
    extern __shared__ float smem[];
    const int VH = H * maps;
    float* qs = smem;
    float* raw = qs + VH * dim;
    float* wt = raw + VH * 64;
    float* run_m = wt + VH * 64;
    float* run_l = run_m + VH;
    float* corr = run_l + VH;
    float* acc = corr + VH;
    float* lam = acc + VH * vdim;
    const int t = rows != nullptr ? rows[blockIdx.x] : (int)blockIdx.x;
    if (t < 0) return;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int p = pos[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int keep = lo < keep_first ? lo : keep_first;     // kept keys below the window's edge: 0 .. keep - 1
    const int* bt = block_tables + (size_t)seg[t] * max_blocks;
    const T* qrow = q + (size_t)t * VH * dim;
    const int per = H / G;
    for (int i = tid; i < VH * dim; i += 256) qs[i] = to_f32(qrow[i]);
    for (int i = tid; i < VH; i += 256) { run_m[i] = -INFINITY; run_l[i] = 0.f; }
    for (int i = tid; i < VH * vdim; i += 256) acc[i] = 0.f;
    if (wave == 0 && maps == 2) {
        float a = 0.f, b = 0.f;
        for (int e = lane; e < dim; e += 64) {
            a = fmaf(to_f32(lq1[e]), to_f32(lk1[e]), a);
            b = fmaf(to_f32(lq2[e]), to_f32(lk2[e]), b);
        }
        a = wave_sum(a);
        b = wave_sum(b);
        if (lane == 0) lam[0] = expf(a) - expf(b) + diff;
    }
    __syncthreads();
    const int pieces = (per + AM_R - 1) / AM_R;
    for (int tile = 0; tile <= (p >> 6); ++tile) {
        const int k0 = tile << 6;
        if (k0 + 63 < lo && k0 >= keep) continue;            // nothing of this tile is seen
        const int key = k0 + lane;
        const bool valid = key <= p && (key >= lo || key < keep);
        // 1. raw scores: a wave takes (group, map, piece) items in turn, a lane a key
        for (int item = wave; item < G * maps * pieces; item += 4) {
            const int g = item / (maps * pieces), m = (item / pieces) % maps, h0 = g * per + (item % pieces) * AM_R;
            const int hn = min(AM_R, (g + 1) * per - h0);
            float dot[AM_R];
#pragma unroll
            for (int r = 0; r < AM_R; ++r) dot[r] = 0.f;
            if (valid) {
                const int pg = bt[key / page];
                const T* krow = kc + (((size_t)pg * G + g) * page + (key % page)) * d + (size_t)m * dim;
                for (int i = 0; i < dim; ++i) {
                    const float kv = to_f32(krow[i]);
#pragma unroll
                    for (int r = 0; r < AM_R; ++r)
                        if (r < hn) dot[r] = fmaf(qs[((h0 + r) * maps + m) * dim + i], kv, dot[r]);
                }
            }
#pragma unroll
            for (int r = 0; r < AM_R; ++r)
                if (r < hn) raw[((h0 + r) * maps + m) * 64 + lane] = dot[r] * scale;
        }
        __syncthreads();
        // 2. running maximum and sum, the tile's weights: a wave takes (head, map) in turn
        for (int h = wave; h < VH; h += 4) {
            const float s = valid ? raw[h * 64 + lane] : -INFINITY;
            const float m_old = run_m[h];
            const float m_new = fmaxf(m_old, wave_max(s));
            const float pj = valid ? expf(s - m_new) : 0.f;
            const float cf = expf(m_old - m_new);
            const float l_new = run_l[h] * cf + wave_sum(pj);
            wt[h * 64 + lane] = pj;
            if (lane == 0) { run_m[h] = m_new; run_l[h] = l_new; corr[h] = cf; }
        }
        __syncthreads();
        // 3. outputs: a thread takes (head, map, value entry) items in turn and walks the tile's seen keys in ascending order:
        //    the kept ones [a0, a1], then the window's [b0, b1]
        const int a0 = 0, a1 = min(63, keep - 1 - k0);
        const int b0 = max(max(lo - k0, 0), a1 + 1), b1 = min(63, p - k0);
        for (int idx = tid; idx < VH * vdim; idx += 256) {
            const int h = idx / vdim, e = idx % vdim, g = (h / maps) / per;
            float a = acc[idx] * corr[h];
            const float* wrow = wt + h * 64;
            for (int j = a0; j <= a1; ++j) {
                const int kk = k0 + j;
                a = fmaf(wrow[j], to_f32(vc[(((size_t)bt[kk / page] * G + g) * d + e) * page + (kk % page)]), a);
            }
            for (int j = b0; j <= b1; ++j) {
                const int kk = k0 + j;
                a = fmaf(wrow[j], to_f32(vc[(((size_t)bt[kk / page] * G + g) * d + e) * page + (kk % page)]), a);
            }
            acc[idx] = a;
        }
        __syncthreads();
    }
    // the denominators' extra term, the division
    for (int idx = tid; idx < VH * vdim; idx += 256) {
        const int h = idx / vdim;
        float L = run_l[h];
        if (sink != nullptr) L += expf(sink[h / maps] - run_m[h]);
        acc[idx] = acc[idx] / L;
    }
    __syncthreads();
    T* orow = out + (size_t)t * out_stride;
    if (maps == 1) {
        for (int idx = tid; idx < H * vdim; idx += 256) orow[idx] = from_f32<T>(acc[idx]);
        return;
    }
    // two maps: a wave takes heads in turn; o = a_0 - lambda a_1, its root mean square, the scale
    const float lambda = lam[0];
    for (int h = wave; h < H; h += 4) {
        const float* a0p = acc + (size_t)(h * 2) * vdim;
        const float* a1p = a0p + vdim;
        float ss = 0.f;
        for (int e = lane; e < vdim; e += 64) {
            const float o = a0p[e] - lambda * a1p[e];
            ss = fmaf(o, o, ss);
        }
        ss = wave_sum(ss);
        const float f = norm_eps >= 0.f ? out_scale / sqrtf(ss / (float)vdim + norm_eps) : out_scale;
        for (int e = lane; e < vdim; e += 64) orow[(size_t)h * vdim + e] = from_f32<T>((a0p[e] - lambda * a1p[e]) * f);
    }
}

extern "C" long ilm_attn_maps_lds_bytes(int H, int maps, int dim, int vdim) {
    const long VH = (long)H * maps;
    return (long)sizeof(float) * (VH * dim + 2L * VH * 64 + 3L * VH + VH * vdim + 4);
}

// rows: null (every token of the step) or a list of n_rows row numbers (-1: no row); out [T, >= H vdim]
extern "C" int ilm_attn_maps(void* out, const void* q, const void* kc, const void* vc, const void* block_tables, const void* seg,
                             const void* pos, const void* rows, int n_rows, int H, int G, int maps, int dim, int vdim, int d, int page,
                             int max_blocks, int out_stride, float scale, int window, int keep_first, const void* sink, const void* lq1,
                             const void* lk1, const void* lq2, const void* lk2, float diff, float norm_eps, float out_scale, int dtype,
                             int w_dt, hipStream_t stream) {
    ILM_REQUIRE(n_rows > 0 && H > 0 && G > 0 && dim > 0 && vdim > 0 && page > 0 && max_blocks > 0, "attn_maps: bad sizes");
    ILM_REQUIRE(H % G == 0, "attn_maps: %d query heads do not divide into %d groups", H, G);
    ILM_REQUIRE(maps == 1 || maps == 2, "attn_maps: %d maps (1 or 2)", maps);
    ILM_REQUIRE(maps * dim <= d && vdim <= d && out_stride >= H * vdim, "attn_maps: %d maps of %d / values of %d in cache heads of %d", maps,
                dim, vdim, d);
    ILM_REQUIRE(maps == 1 || (lq1 && lk1 && lq2 && lk2), "attn_maps: two maps need the four vectors of their weight");
    ILM_REQUIRE(window >= 0 && keep_first >= 0, "attn_maps: window %d, kept first tokens %d", window, keep_first);
    const long shm = ilm_attn_maps_lds_bytes(H, maps, dim, vdim);
    ILM_REQUIRE(shm <= 160 * 1024 - 1024, "attn_maps: %d heads x %d maps of %d / %d need %ld bytes of LDS, more than a compute unit has", H,
                maps, dim, vdim, shm);
#define AM_LAUNCH(T_, TW_)                                                                                                  \
    {                                                                                                                       \
        auto kern = attn_maps_kernel<T_, TW_>;                                                                              \
        if (shm > 48 * 1024) {                                                                                              \
            hipError_t e_ = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm);   \
            ILM_REQUIRE(e_ == hipSuccess, "attn_maps: %ld bytes of LDS refused: %s", shm, hipGetErrorString(e_));            \
        }                                                                                                                   \
        kern<<<n_rows, 256, shm, stream>>>((T_*)out, (const T_*)q, (const T_*)kc, (const T_*)vc, (const int*)block_tables,   \
                                           (const int*)seg, (const int*)pos, (const int*)rows, H, G, maps, dim, vdim, d,    \
                                           page, max_blocks, out_stride, scale, window, keep_first, (const float*)sink,     \
                                           (const TW_*)lq1, (const TW_*)lk1, (const TW_*)lq2, (const TW_*)lk2, diff,        \
                                           norm_eps, out_scale);                                                            \
    }
    if (dtype == ILM_DTYPE_F32 && w_dt == ILM_DTYPE_F32) AM_LAUNCH(float, float)
    else if (dtype == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_BF16) AM_LAUNCH(bf16, bf16)
    else if (dtype == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_F32) AM_LAUNCH(bf16, float)
    else ILM_REQUIRE(false, "attn_maps: dtypes %d / %d", dtype, w_dt);
#undef AM_LAUNCH
    ILM_LAUNCH_CHECK("attn_maps");
    return 0;
}

// ------------------------------------------------------------------------------------------
// One wave a (token, head): o = a_0 - lambda a_1 over vdim entries of float rows [T, H 2, d], normed and scaled.
// ------------------------------------------------------------------------------------------
template <typename T, typename TW>
__global__ void __launch_bounds__(256)
maps_combine_kernel(T* __restrict__ out, const float* __restrict__ a, int T_, int H, int vdim, int d, int out_stride,
                    const TW* __restrict__ lq1, const TW* __restrict__ lk1, const TW* __restrict__ lq2, const TW* __restrict__ lk2,
                    float diff, float norm_eps, float out_scale, int dim) {
    const int lane = threadIdx.x & 63;
    const long item = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= (long)T_ * H) return;
    const int t = (int)(item / H), h = (int)(item % H);
    float x = 0.f, y = 0.f;
    for (int e = lane; e < dim; e += 64) {
        x = fmaf(to_f32(lq1[e]), to_f32(lk1[e]), x);
        y = fmaf(to_f32(lq2[e]), to_f32(lk2[e]), y);
    }
    const float lambda = expf(wave_sum(x)) - expf(wave_sum(y)) + diff;
    const float* a0 = a + ((size_t)t * H + h) * 2 * d;
    const float* a1 = a0 + d;
    float ss = 0.f;
    for (int e = lane; e < vdim; e += 64) {
        const float o = a0[e] - lambda * a1[e];
        ss = fmaf(o, o, ss);
    }
    ss = wave_sum(ss);
    const float f = norm_eps >= 0.f ? out_scale / sqrtf(ss / (float)vdim + norm_eps) : out_scale;
    T* orow = out + (size_t)t * out_stride + (size_t)h * vdim;
    for (int e = lane; e < vdim; e += 64) orow[e] = from_f32<T>((a0[e] - lambda * a1[e]) * f);
}

extern "C" int ilm_maps_combine(void* out, const void* a, int T_, int H, int vdim, int d, int out_stride, const void* lq1, const void* lk1,
                                const void* lq2, const void* lk2, float diff, float norm_eps, float out_scale, int dim, int w_dt,
                                hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && H > 0 && vdim > 0 && vdim <= d && dim > 0 && out_stride >= H * vdim, "maps_combine: bad sizes");
    ILM_REQUIRE(lq1 && lk1 && lq2 && lk2, "maps_combine: the four vectors of the maps' weight are needed");
    const unsigned blocks = (unsigned)(((long)T_ * H + 3) / 4);
    if (w_dt == ILM_DTYPE_BF16)
        maps_combine_kernel<bf16, bf16><<<blocks, 256, 0, stream>>>((bf16*)out, (const float*)a, T_, H, vdim, d, out_stride, (const bf16*)lq1,
                                                                   (const bf16*)lk1, (const bf16*)lq2, (const bf16*)lk2, diff, norm_eps,
                                                                   out_scale, dim);
    else if (w_dt == ILM_DTYPE_F32)
        maps_combine_kernel<bf16, float><<<blocks, 256, 0, stream>>>((bf16*)out, (const float*)a, T_, H, vdim, d, out_stride, (const float*)lq1,
                                                                    (const float*)lk1, (const float*)lq2, (const float*)lk2, diff, norm_eps,
                                                                    out_scale, dim);
    else
        ILM_REQUIRE(false, "maps_combine: dtype %d", w_dt);
    ILM_LAUNCH_CHECK("maps_combine");
    return 0;
}
