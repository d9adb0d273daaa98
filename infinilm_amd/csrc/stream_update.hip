// Kernels around a residual stream whose sublayers' results are changed on their way into it:
//
//   ilm_embed_pos       r[t] = scale * E[ids[t]] + P[pos[t]]: token row plus a learned row of the position, float32.
//   ilm_stream_update   r[t] += alpha * f(y[t]) for a branch y (bf16/float rows, or float32 parts of a K-split product that are
//                       summed first) where f is
//                         SU_PLAIN  y
//                         SU_GATED  y * sigmoid(z + zb)         z [T, H] a second product's rows, zb [H] its bias (or none)
//                         SU_NORMED y / rms(y) * bw             the branch's own RMS norm with a weight (eps inside the root)
//                       and then, if an output is asked for, x[t] = r[t] normed in `groups` consecutive equal parts (each by its
//                       own root mean square) times a weight; without a weight x is r in the output's dtype (for a product that
//                       reads the stream itself).  A block a row; the row stays in LDS between the sums and the result.
//   ilm_embed_gate      g[t, j] = gelu_tanh(z[t, j]) * E[ids[t], col0 + j]: a slice of a second embedding table, gated.
//   ilm_softcap         x = cap * tanh(x / cap) in place on float32.
#include "common.h"

#define SU_NONE 0
#define SU_PLAIN 1
#define SU_GATED 2
#define SU_NORMED 3
#define SU_THREADS 256
#define SU_MAX_H 12288
#define SU_MAX_GROUPS 256

__device__ __forceinline__ float ld_any(const void* p, size_t i, int dt) {
    return dt == ILM_DTYPE_F32 ? ((const float*)p)[i] : bf16_bits_to_f32(((const uint16_t*)p)[i]);
}
__device__ __forceinline__ void st_any(void* p, size_t i, int dt, float v) {
    if (dt == ILM_DTYPE_F32) ((float*)p)[i] = v;
    else ((bf16*)p)[i] = from_f32<bf16>(v);
}

__global__ void embed_pos_kernel(float* __restrict__ r, const int* __restrict__ ids, const int* __restrict__ pos,
                                 const void* __restrict__ table, const void* __restrict__ ptable, int H, float scale, int dt) {
    const int t = blockIdx.x;
    const size_t a = (size_t)ids[t] * H, b = (size_t)pos[t] * H;
    float* out = r + (size_t)t * H;
    for (int j = threadIdx.x; j < H; j += blockDim.x) out[j] = scale * ld_any(table, a + j, dt) + ld_any(ptable, b + j, dt);
}

extern "C" int ilm_embed_pos(void* r, const void* ids, const void* pos, const void* table, const void* ptable, int T_, int H, int V,
                             int P, float scale, int dtype, hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && H > 0 && V > 0 && P > 0, "embed_pos: bad sizes T=%d H=%d V=%d P=%d", T_, H, V, P);
    ILM_REQUIRE(dtype == ILM_DTYPE_F32 || dtype == ILM_DTYPE_BF16, "embed_pos: unknown dtype %d", dtype);
    embed_pos_kernel<<<T_, 256, 0, stream>>>((float*)r, (const int*)ids, (const int*)pos, table, ptable, H, scale, dtype);
    ILM_LAUNCH_CHECK("embed_pos");
    return 0;
}

__device__ __forceinline__ float su_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }

__global__ void __launch_bounds__(SU_THREADS)
stream_update_kernel(void* __restrict__ x, float* __restrict__ r, const void* __restrict__ y, const void* __restrict__ z,
                     const void* __restrict__ zb, const void* __restrict__ bw, const void* __restrict__ w, int H, int groups, int kind,
                     float alpha, float eps_b, float eps, int x_dt, int y_dt, int z_dt, int w_dt, int parts, size_t part_stride,
                     int y_stride, int z_stride) {
    extern __shared__ float row[];          // H floats
    __shared__ float red[SU_THREADS / 64];
    __shared__ float rstd_g[SU_MAX_GROUPS];
    const int t = blockIdx.x, tid = threadIdx.x;
    float* rr = r + (size_t)t * H;
    if (kind == SU_NONE) {
        for (int j = tid; j < H; j += SU_THREADS) row[j] = rr[j];
    } else {
        // the branch's row (parts summed in order)
        float ss = 0.f;
        for (int j = tid; j < H; j += SU_THREADS) {
            float v = 0.f;
            for (int p = 0; p < parts; ++p) v += ld_any(y, (size_t)p * part_stride + (size_t)t * y_stride + j, y_dt);
            row[j] = v;
            ss = fmaf(v, v, ss);
        }
        float f = alpha;
        if (kind == SU_NORMED) f = alpha / sqrtf(block_sum<SU_THREADS / 64>(ss, red) / (float)H + eps_b);
        for (int j = tid; j < H; j += SU_THREADS) {
            float v = row[j] * f;
            if (kind == SU_GATED) {
                float g = ld_any(z, (size_t)t * z_stride + j, z_dt);
                if (zb != nullptr) g += ld_any(zb, j, w_dt);
                v *= su_sigmoid(g);
            } else if (kind == SU_NORMED) {
                v *= ld_any(bw, j, w_dt);
            }
            const float s = rr[j] + v;
            rr[j] = s;
            row[j] = s;
        }
    }
    if (x == nullptr) return;
    if (w == nullptr) {
        for (int j = tid; j < H; j += SU_THREADS) st_any(x, (size_t)t * H + j, x_dt, row[j]);
        return;
    }
    __syncthreads();
    const int gs = H / groups, wave = tid >> 6, lane = tid & 63;
    for (int g = wave; g < groups; g += SU_THREADS / 64) {
        float ss = 0.f;
        for (int j = lane; j < gs; j += 64) {
            const float v = row[g * gs + j];
            ss = fmaf(v, v, ss);
        }
        ss = wave_sum(ss);
        if (lane == 0) rstd_g[g] = 1.0f / sqrtf(ss / (float)gs + eps);
    }
    __syncthreads();
    for (int j = tid; j < H; j += SU_THREADS) st_any(x, (size_t)t * H + j, x_dt, row[j] * rstd_g[j / gs] * ld_any(w, j, w_dt));
}


// ---- the same with four elements a thread (rows, strides and pointers that allow 16-byte float and 8-byte bfloat16 accesses) ----
__device__ __forceinline__ float4 ld4_any(const void* p, size_t i, int dt) {
    if (dt == ILM_DTYPE_F32) return *reinterpret_cast<const float4*>((const float*)p + i);
    const uint2 v = *reinterpret_cast<const uint2*>((const uint16_t*)p + i);
    return make_float4(bf16_bits_to_f32((uint16_t)(v.x & 0xffffu)), bf16_bits_to_f32((uint16_t)(v.x >> 16)),
                       bf16_bits_to_f32((uint16_t)(v.y & 0xffffu)), bf16_bits_to_f32((uint16_t)(v.y >> 16)));
}
__device__ __forceinline__ void st4_any(void* p, size_t i, int dt, float4 v) {
    if (dt == ILM_DTYPE_F32) {
        *reinterpret_cast<float4*>((float*)p + i) = v;
    } else {
        uint2 o;
        o.x = (uint32_t)from_f32<bf16>(v.x).bits | ((uint32_t)from_f32<bf16>(v.y).bits << 16);
        o.y = (uint32_t)from_f32<bf16>(v.z).bits | ((uint32_t)from_f32<bf16>(v.w).bits << 16);
        *reinterpret_cast<uint2*>((uint16_t*)p + i) = o;
    }
}

template <int THREADS>
__global__ void __launch_bounds__(THREADS)
stream_update_vec_kernel(void* __restrict__ x, float* __restrict__ r, const void* __restrict__ y, const void* __restrict__ z,
                         const void* __restrict__ zb, const void* __restrict__ bw, const void* __restrict__ w, int H, int groups, int kind,
                         float alpha, float eps_b, float eps, int x_dt, int y_dt, int z_dt, int w_dt, int parts, size_t part_stride,
                         int y_stride, int z_stride) {
    extern __shared__ float4 row4[];         // H floats
    float* row = reinterpret_cast<float*>(row4);
    __shared__ float red[THREADS / 64];
    __shared__ float rstd_g[SU_MAX_GROUPS];
    const int t = blockIdx.x, tid = threadIdx.x;
    float* rr = r + (size_t)t * H;
    if (kind == SU_NONE) {
        for (int j = tid * 4; j < H; j += THREADS * 4) *reinterpret_cast<float4*>(&row[j]) = *reinterpret_cast<const float4*>(&rr[j]);
    } else {
        float ss = 0.f;
        for (int j = tid * 4; j < H; j += THREADS * 4) {
            float4 v = ld4_any(y, (size_t)t * y_stride + j, y_dt);
            for (int p = 1; p < parts; ++p) {
                const float4 a = ld4_any(y, (size_t)p * part_stride + (size_t)t * y_stride + j, y_dt);
                v.x += a.x, v.y += a.y, v.z += a.z, v.w += a.w;
            }
            *reinterpret_cast<float4*>(&row[j]) = v;
            ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ss))));
        }
        float f = alpha;
        if (kind == SU_NORMED) f = alpha / sqrtf(block_sum<THREADS / 64>(ss, red) / (float)H + eps_b);
        for (int j = tid * 4; j < H; j += THREADS * 4) {
            float4 v = *reinterpret_cast<const float4*>(&row[j]);
            v.x *= f, v.y *= f, v.z *= f, v.w *= f;
            if (kind == SU_GATED) {
                float4 g = ld4_any(z, (size_t)t * z_stride + j, z_dt);
                if (zb != nullptr) {
                    const float4 b = ld4_any(zb, j, w_dt);
                    g.x += b.x, g.y += b.y, g.z += b.z, g.w += b.w;
                }
                v.x *= su_sigmoid(g.x), v.y *= su_sigmoid(g.y), v.z *= su_sigmoid(g.z), v.w *= su_sigmoid(g.w);
            } else if (kind == SU_NORMED) {
                const float4 b = ld4_any(bw, j, w_dt);
                v.x *= b.x, v.y *= b.y, v.z *= b.z, v.w *= b.w;
            }
            float4 s = *reinterpret_cast<const float4*>(&rr[j]);
            s.x += v.x, s.y += v.y, s.z += v.z, s.w += v.w;
            *reinterpret_cast<float4*>(&rr[j]) = s;
            *reinterpret_cast<float4*>(&row[j]) = s;
        }
    }
    if (x == nullptr) return;
    if (w == nullptr) {
        for (int j = tid * 4; j < H; j += THREADS * 4) st4_any(x, (size_t)t * H + j, x_dt, *reinterpret_cast<const float4*>(&row[j]));
        return;
    }
    __syncthreads();
    const int gs = H / groups, wave = tid >> 6, lane = tid & 63;
    for (int g = wave; g < groups; g += THREADS / 64) {
        float ss = 0.f;
        for (int j = lane; j < gs; j += 64) {
            const float v = row[g * gs + j];
            ss = fmaf(v, v, ss);
        }
        ss = wave_sum(ss);
        if (lane == 0) rstd_g[g] = 1.0f / sqrtf(ss / (float)gs + eps);
    }
    __syncthreads();
    for (int j = tid * 4; j < H; j += THREADS * 4) {
        float4 v = *reinterpret_cast<const float4*>(&row[j]);
        const float4 ww = ld4_any(w, j, w_dt);
        v.x *= rstd_g[j / gs] * ww.x, v.y *= rstd_g[(j + 1) / gs] * ww.y, v.z *= rstd_g[(j + 2) / gs] * ww.z, v.w *= rstd_g[(j + 3) / gs] * ww.w;
        st4_any(x, (size_t)t * H + j, x_dt, v);
    }
}

static bool su_aligned(const void* p, int dt) { return p == nullptr || ((uintptr_t)p % (dt == ILM_DTYPE_F32 ? 16 : 8)) == 0; }

extern "C" int ilm_stream_update(void* x, void* r, const void* y, const void* z, const void* zb, const void* bw, const void* w,
                                 int rows, int H, int groups, int kind, float alpha, float eps_b, float eps, int x_dt, int y_dt,
                                 int z_dt, int w_dt, int parts, long part_stride, int y_stride, int z_stride, hipStream_t stream) {
    ILM_REQUIRE(rows > 0 && H > 0 && H <= SU_MAX_H, "stream_update: %d rows of %d (at most %d)", rows, H, SU_MAX_H);
    ILM_REQUIRE(kind >= SU_NONE && kind <= SU_NORMED, "stream_update: unknown kind %d", kind);
    ILM_REQUIRE(kind == SU_NONE || (y != nullptr && parts >= 1), "stream_update: a branch is missing");
    ILM_REQUIRE(kind != SU_GATED || z != nullptr, "stream_update: a gated branch needs the gate's rows");
    ILM_REQUIRE(kind != SU_NORMED || bw != nullptr, "stream_update: a normed branch needs the norm's weight");
    ILM_REQUIRE(w == nullptr || (groups >= 1 && groups <= SU_MAX_GROUPS && H % groups == 0),
                "stream_update: rows of %d do not divide into %d groups (at most %d)", H, groups, SU_MAX_GROUPS);
    ILM_REQUIRE(w == nullptr || x != nullptr, "stream_update: a norm needs an output");
    const bool vec = H % 4 == 0 && y_stride % 4 == 0 && z_stride % 4 == 0 && part_stride % 4 == 0 && su_aligned(x, x_dt) && su_aligned(r, ILM_DTYPE_F32) &&
                     su_aligned(y, y_dt) && su_aligned(z, z_dt) && su_aligned(zb, w_dt) && su_aligned(bw, w_dt) && su_aligned(w, w_dt);
#define SU_ARGS x, (float*)r, y, z, zb, bw, w, H, groups < 1 ? 1 : groups, kind, alpha, eps_b, eps, x_dt, y_dt, z_dt, w_dt, parts, \
                (size_t)part_stride, y_stride, z_stride
    // (a row of up to 1,024 numbers gives 256 threads four each; wider rows of a launch that leaves compute units idle take 1,024 threads)
    if (vec && H > 1024 && rows <= 2 * ilm_num_cus())
        stream_update_vec_kernel<1024><<<rows, 1024, (size_t)H * sizeof(float), stream>>>(SU_ARGS);
    else if (vec)
        stream_update_vec_kernel<256><<<rows, 256, (size_t)H * sizeof(float), stream>>>(SU_ARGS);
    else
        stream_update_kernel<<<rows, SU_THREADS, (size_t)H * sizeof(float), stream>>>(SU_ARGS);
#undef SU_ARGS
    ILM_LAUNCH_CHECK("stream_update");
    return 0;
}

__device__ __forceinline__ float su_gelu_tanh(float v) {
    const float u = 0.7978845608028654f * (v + 0.044715f * v * v * v);
    return 0.5f * v * (1.0f + tanhf(u));
}

__global__ void embed_gate_kernel(void* __restrict__ g, const void* __restrict__ z, const int* __restrict__ ids,
                                  const void* __restrict__ table, int n, int table_stride, int col0, int z_stride, int dt, int total) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int t = i / n, j = i % n;
    const float e = ld_any(table, (size_t)ids[t] * table_stride + col0 + j, dt);
    st_any(g, (size_t)t * n + j, dt, su_gelu_tanh(ld_any(z, (size_t)t * z_stride + j, dt)) * e);
}

extern "C" int ilm_embed_gate(void* g, const void* z, const void* ids, const void* table, int T_, int n, int table_stride, int col0,
                              int z_stride, int dtype, hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && n > 0 && col0 >= 0 && col0 + n <= table_stride, "embed_gate: columns %d .. %d of %d", col0, col0 + n,
                table_stride);
    ILM_REQUIRE((long)T_ * n < (1L << 31), "embed_gate: too many elements");
    ILM_REQUIRE(dtype == ILM_DTYPE_F32 || dtype == ILM_DTYPE_BF16, "embed_gate: unknown dtype %d", dtype);
    const int total = T_ * n;
    embed_gate_kernel<<<(total + 255) / 256, 256, 0, stream>>>(g, z, (const int*)ids, table, n, table_stride, col0, z_stride, dtype, total);
    ILM_LAUNCH_CHECK("embed_gate");
    return 0;
}

__global__ void softcap_kernel(float* __restrict__ x, long n, float cap, float inv) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] = cap * tanhf(x[i] * inv);
}

extern "C" int ilm_softcap(void* x, long n, float cap, hipStream_t stream) {
    ILM_REQUIRE(n > 0 && cap > 0.f, "softcap: %ld numbers, cap %g", n, (double)cap);
    softcap_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>((float*)x, n, cap, 1.0f / cap);
    ILM_LAUNCH_CHECK("softcap");
    return 0;
}
