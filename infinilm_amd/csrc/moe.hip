// A feed-forward of many small experts of which every token uses a few.
//
//   ilm_moe_route     per token: the `top` largest of E router logits (ties to the lower index), their indices and as weights
//                     a scale times sigmoid(logit) or the logit's softmax over all E experts; one wave a token, all float32.
//   ilm_moe_sort      the (token, slot) pairs of a step ordered by expert: offsets per expert, the pair at every sorted
//                     place and the place of every pair, and the list of row tiles (expert, first place, rows) that the
//                     products below walk.  One block; the order inside an expert is whatever the atomics give, which no
//                     row's result depends on.
//   ilm_moe_gemm      for every tile of rows of one expert e: out[place] = f(W_e x[place]) with
//                       GLU form    x = weight(pair) * h[token of the pair], W_e = [gate rows | up rows],
//                                   g = min(gate, limit), u = clamp(up, -limit, limit), out = g sigmoid(alpha g) (u + 1)
//                       plain form  x = rows in sorted order (or, with the list of pairs, the pairs' token rows), out = W_e x
//                                   or the square of relu(W_e x)
//                     bfloat16 on v_mfma_f32_16x16x32_bf16 (tiles of 64 rows x 64 outputs, operands through LDS in steps of
//                     64 k, the next step's loads in flight), float32 and odd sizes by FMA in ascending k.
//   ilm_moe_combine   y[t] = sum over the token's slots of (weight of the pair *) out[place of (t, slot)] (+ shared[t] * sigmoid(sg[t])).
//   ilm_glu_clamp     the experts' activation on fused [gate | up] rows of a dense product.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define MOE_MAX_E 1024
#define MOE_TM 64
#define MOE_BM 128  // rows of a tile of the many-rows kernel
#define MOE_BGROUP 4 // row tiles of that kernel that walk the output slices together
#define MOE_TN 64
#define MOE_KS 64
#define MOE_LD (MOE_KS + 8)   // bf16 elements a row of a tile in LDS (144 bytes)

__device__ __forceinline__ float moe_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }

// ---- routing -------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
moe_route_kernel(int* __restrict__ ids, float* __restrict__ wts, const float* __restrict__ z, int T_, int E, int top, int z_stride,
                 int softmax, float wscale) {
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (t >= T_) return;
    float v[MOE_MAX_E / 64];
#pragma unroll
    for (int i = 0; i < MOE_MAX_E / 64; ++i) {
        const int e = lane + 64 * i;
        v[i] = e < E ? z[(size_t)t * z_stride + e] : -INFINITY;
    }
    // softmax weights: the row's maximum and the sum of exponentials over all experts, in lane order
    float zmax = -INFINITY, zsum = 0.f;
    if (softmax) {
#pragma unroll
        for (int i = 0; i < MOE_MAX_E / 64; ++i) zmax = fmaxf(zmax, v[i]);
        zmax = wave_max(zmax);
#pragma unroll
        for (int i = 0; i < MOE_MAX_E / 64; ++i)
            if (lane + 64 * i < E) zsum += expf(v[i] - zmax);
        zsum = wave_sum(zsum);
    }
    for (int s = 0; s < top; ++s) {
        float best = -INFINITY;
        int bi = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < MOE_MAX_E / 64; ++i) {
            const int e = lane + 64 * i;
            if (e < E && (v[i] > best || (v[i] == best && e < bi))) {
                best = v[i];
                bi = e;
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(best, o, 64);
            const int oi = __shfl_xor(bi, o, 64);
            if (ov > best || (ov == best && oi < bi)) {
                best = ov;
                bi = oi;
            }
        }
        if (bi >= E) bi = s;       // nothing compared larger (a row of NaNs): any valid expert, so that no index downstream is unset
        if (lane == 0) {
            ids[(size_t)t * top + s] = bi;
            wts[(size_t)t * top + s] = wscale * (softmax ? expf(best - zmax) / zsum : moe_sigmoid(best));
        }
#pragma unroll
        for (int i = 0; i < MOE_MAX_E / 64; ++i)
            if (lane + 64 * i == bi) v[i] = -INFINITY;
    }
}

extern "C" int ilm_moe_route(void* ids, void* wts, const void* z, int T_, int E, int top, int z_stride, int softmax, float wscale,
                             hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && E > 0 && E <= MOE_MAX_E && top > 0 && top <= E, "moe_route: %d tokens, %d experts (at most %d), top %d", T_, E,
                MOE_MAX_E, top);
    moe_route_kernel<<<(T_ + 3) / 4, 256, 0, stream>>>((int*)ids, (float*)wts, (const float*)z, T_, E, top, z_stride, softmax, wscale);
    ILM_LAUNCH_CHECK("moe_route");
    return 0;
}

// ---- ordering by expert --------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(1024)
moe_sort_kernel(int* __restrict__ offsets, int* __restrict__ perm, int* __restrict__ inv, int* __restrict__ tiles, int* __restrict__ n_tiles,
                const int* __restrict__ ids, int P, int E, int max_tiles, int tile_rows) {
    __shared__ int cnt[MOE_MAX_E], cur[MOE_MAX_E], tbase[MOE_MAX_E];
    const int tid = threadIdx.x;
    for (int e = tid; e < E; e += 1024) cnt[e] = 0;
    __syncthreads();
    for (int p = tid; p < P; p += 1024) {
        const int e = ids[p];
        if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
    }
    __syncthreads();
    if (tid == 0) {
        int off = 0, tb = 0;
        for (int e = 0; e < E; ++e) {
            offsets[e] = off;
            cur[e] = off;
            tbase[e] = tb;
            off += cnt[e];
            tb += (cnt[e] + tile_rows - 1) / tile_rows;
        }
        offsets[E] = off;
        *n_tiles = tb < max_tiles ? tb : max_tiles;
    }
    __syncthreads();
    for (int e = tid; e < E; e += 1024) {
        const int n = cnt[e], base = cur[e];
        for (int i = 0, tb = tbase[e]; i < n && tb < max_tiles; i += tile_rows, ++tb) {
            tiles[3 * tb] = e;
            tiles[3 * tb + 1] = base + i;
            tiles[3 * tb + 2] = n - i < tile_rows ? n - i : tile_rows;
        }
    }
    __syncthreads();
    for (int p = tid; p < P; p += 1024) {
        const int e = ids[p];
        if (e >= 0 && e < E) {
            const int at = atomicAdd(&cur[e], 1);
            perm[at] = p;
            inv[p] = at;
        }
    }
}

extern "C" int ilm_moe_tile_rows() { return MOE_TM; }

extern "C" int ilm_moe_sort(void* offsets, void* perm, void* inv, void* tiles, void* n_tiles, const void* ids, int P, int E,
                            int max_tiles, int tile_rows, hipStream_t stream) {
    ILM_REQUIRE(P > 0 && E > 0 && E <= MOE_MAX_E, "moe_sort: %d pairs, %d experts (at most %d)", P, E, MOE_MAX_E);
    ILM_REQUIRE(tile_rows == MOE_TM || tile_rows == MOE_BM, "moe_sort: tiles of %d rows (%d or %d)", tile_rows, MOE_TM, MOE_BM);
    const int need = P / tile_rows + (E < P ? E : P);
    ILM_REQUIRE(max_tiles >= (need < P ? need : P), "moe_sort: %d tiles do not hold %d pairs of %d experts", max_tiles, P, E);
    moe_sort_kernel<<<1, 1024, 0, stream>>>((int*)offsets, (int*)perm, (int*)inv, (int*)tiles, (int*)n_tiles, (const int*)ids, P, E, max_tiles, tile_rows);
    ILM_LAUNCH_CHECK("moe_sort");
    return 0;
}

// ---- the experts' products -----------------------------------------------------------------------------------------
__device__ __forceinline__ float moe_glu(float g, float u, float limit, float alpha) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g * moe_sigmoid(alpha * g) * (u + 1.0f);
}

// 8 bfloat16 times a float, rounded back
__device__ __forceinline__ uint4 moe_scale8(uint4 v, float w) {
    uint32_t in[4] = {v.x, v.y, v.z, v.w}, out[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float lo = bf16_bits_to_f32((uint16_t)(in[i] & 0xffffu)) * w, hi = bf16_bits_to_f32((uint16_t)(in[i] >> 16)) * w;
        out[i] = (uint32_t)from_f32<bf16>(lo).bits | ((uint32_t)from_f32<bf16>(hi).bits << 16);
    }
    return make_uint4(out[0], out[1], out[2], out[3]);
}

// bfloat16 on the matrix cores.  Block: 4 waves; tile: up to 64 rows of one expert x 64 outputs (GLU: 64 gate + 64 up rows of
// W); wave w owns outputs 16 w .. 16 w + 15 for all four groups of 16 rows.  K % 8 == 0, rows 16-byte aligned.
// PAIR (plain form): a workgroup takes two blocks of 64 outputs (128 rows of W), as the GLU form takes gate and up rows: twice
// the bytes of W in flight a workgroup, which is what a step of few rows an expert (streaming W once) is bound by.
template <bool GLU, bool PAIR = false>
__global__ void __launch_bounds__(256)
moe_gemm_mfma_kernel(bf16* __restrict__ out, int ld_out, const bf16* __restrict__ X, int ldx, const int* __restrict__ perm, int top,
                     const float* __restrict__ pair_w, const bf16* __restrict__ W, size_t w_expert, int ldw, const int* __restrict__ tiles,
                     const int* __restrict__ n_tiles, int N, int K, float limit, float alpha, int act) {
    constexpr int WR = (GLU || PAIR) ? 2 : 1;
    constexpr int TNW = PAIR ? 2 * MOE_TN : MOE_TN;     // outputs a workgroup
    __shared__ __attribute__((aligned(16))) bf16 xs[MOE_TM * MOE_LD];
    __shared__ __attribute__((aligned(16))) bf16 ws[WR * MOE_TN * MOE_LD];
    __shared__ int src_row[MOE_TM];
    __shared__ float src_w[MOE_TM];
    const int tile = blockIdx.y;
    if (tile >= *n_tiles) return;
    const int e = tiles[3 * tile], place0 = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
    const int n0 = blockIdx.x * TNW, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    if (tid < MOE_TM) {
        int row = -1;
        float w = 1.0f;
        if (tid < rows) {
            if (GLU || perm != nullptr) {     // rows gathered from the tokens' rows (the plain form: only with a list of pairs)
                const int pair = perm != nullptr ? perm[place0 + tid] : place0 + tid;
                row = pair / top;
                if (pair_w != nullptr) w = pair_w[pair];
            } else {
                row = place0 + tid;
            }
        }
        src_row[tid] = row;
        src_w[tid] = w;
    }
    __syncthreads();
    const bf16* We = W + (size_t)e * w_expert;
    // what this thread loads a step: X rows lr, lr + 32 and W rows lr, lr + 32 (of each half), 16 bytes at k chunk lc
    const int lr = tid >> 3, lc = tid & 7;
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    // Two sets of load registers take the k-steps in turn, so that a step's loads are in flight over two steps' products: a
    // step of few rows an expert streams W once and waits for memory, not for the matrix cores.
#define MOE_LOAD_SET(XR, WRG, K0)                                                                                          \
    {                                                                                                                      \
        const int k = (K0) + lc * 8;                                                                                       \
        const bool kok = k < K;                                                                                            \
        _Pragma("unroll") for (int i = 0; i < 2; ++i) {                                                                    \
            const int r = src_row[lr + 32 * i];                                                                            \
            uint4 v = zero;                                                                                                \
            if (kok && r >= 0) {                                                                                           \
                v = *reinterpret_cast<const uint4*>(X + (size_t)r * ldx + k);                                              \
                /* the pair's score on the rows as they are loaded: with few rows an expert this kernel streams W, and */  \
                /* measured against the score on the float sums (as the many-rows kernel has it) it is the faster one */   \
                /* here (192 against 235 us for 64 tokens x 2 of 16 experts at width 4,096) */                             \
                if (GLU) v = moe_scale8(v, src_w[lr + 32 * i]);                                                            \
            }                                                                                                              \
            XR[i] = v;                                                                                                     \
        }                                                                                                                  \
        _Pragma("unroll") for (int h = 0; h < WR; ++h) _Pragma("unroll") for (int i = 0; i < 2; ++i) {                      \
            const int n = n0 + lr + 32 * i + (PAIR ? h * MOE_TN : 0);                                                      \
            uint4 v = zero;                                                                                                \
            if (kok && n < N) v = *reinterpret_cast<const uint4*>(We + (size_t)((GLU ? h * N : 0) + n) * ldw + k);         \
            WRG[h * 2 + i] = v;                                                                                            \
        }                                                                                                                  \
    }
#define MOE_STAGE_SET(XR, WRG)                                                                                              \
    {                                                                                                                      \
        _Pragma("unroll") for (int i = 0; i < 2; ++i) *reinterpret_cast<uint4*>(&xs[(lr + 32 * i) * MOE_LD + lc * 8]) = XR[i]; \
        _Pragma("unroll") for (int h = 0; h < WR; ++h) _Pragma("unroll") for (int i = 0; i < 2; ++i)                        \
            *reinterpret_cast<uint4*>(&ws[(h * MOE_TN + lr + 32 * i) * MOE_LD + lc * 8]) = WRG[h * 2 + i];                  \
    }
    uint4 xr[2], wr[WR * 2], xr2[2], wr2[WR * 2];
    f32x4 acc[WR][4];
#pragma unroll
    for (int h = 0; h < WR; ++h)
#pragma unroll
        for (int g = 0; g < 4; ++g) acc[h][g] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int r16 = lane & 15, q = lane >> 4;
    const int groups = (rows + 15) >> 4;
    auto compute = [&]() {
#pragma unroll
        for (int ks = 0; ks < MOE_KS / 32; ++ks) {
            uint4 a[WR];
#pragma unroll
            for (int h = 0; h < WR; ++h) a[h] = *reinterpret_cast<const uint4*>(&ws[(h * MOE_TN + wave * 16 + r16) * MOE_LD + ks * 32 + q * 8]);
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                if (g < groups) {
                    const uint4 b = *reinterpret_cast<const uint4*>(&xs[(g * 16 + r16) * MOE_LD + ks * 32 + q * 8]);
#pragma unroll
                    for (int h = 0; h < WR; ++h)
                        acc[h][g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[h]), __builtin_bit_cast(bf16x8, b),
                                                                            acc[h][g], 0, 0, 0);
                }
            }
        }
    };
    MOE_LOAD_SET(xr, wr, 0)
    MOE_LOAD_SET(xr2, wr2, MOE_KS)
    for (int k0 = 0; k0 < K; k0 += 2 * MOE_KS) {
        __syncthreads();           // the last step's readers are done
        MOE_STAGE_SET(xr, wr)
        __syncthreads();
        if (k0 + 2 * MOE_KS < K) MOE_LOAD_SET(xr, wr, k0 + 2 * MOE_KS)
        compute();
        if (k0 + MOE_KS < K) {
            __syncthreads();
            MOE_STAGE_SET(xr2, wr2)
            __syncthreads();
            if (k0 + 3 * MOE_KS < K) MOE_LOAD_SET(xr2, wr2, k0 + 3 * MOE_KS)
            compute();
        }
    }
#undef MOE_LOAD_SET
#undef MOE_STAGE_SET
    // lane holds rows m = 16 g + r16 and outputs n = n0 + 16 wave + 4 q + i
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const int m = g * 16 + r16;
        if (m >= rows) continue;
        bf16* orow = out + (size_t)(place0 + m) * ld_out;
#pragma unroll
        for (int hb = 0; hb < (PAIR ? 2 : 1); ++hb)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int n = n0 + hb * MOE_TN + wave * 16 + q * 4 + i;
                if (n < N) {
                    float v = acc[hb][g][i];
                    if (GLU) v = moe_glu(v, acc[WR - 1][g][i], limit, alpha);
                    else if (act == 1) { v = fmaxf(v, 0.f); v *= v; }
                    orow[n] = from_f32<bf16>(v);
                }
            }
    }
}


// bfloat16 on the matrix cores, many rows an expert.  Block: 2 x WN waves; tile: up to 128 rows of one expert x 64 WN rows of W
// (GLU: the gate rows and the up rows of 32 WN outputs; else 64 WN outputs); wave (wm, wn) owns 64 rows x 64 rows of W (GLU:
// gate and up of 32 outputs, so the activation has both in one thread): 16 products for 8 fragment reads a k-step.  WN = 4
// reads a third fewer bytes a product from the caches than WN = 2 (a tile's operands: 128 + 256 rows for 128 x 256 results).
template <bool GLU, int WN>
// (Three waves a SIMD: left to itself the compiler takes 170 registers a lane, two more than three workgroups a compute unit allow.)
__global__ void __launch_bounds__(128 * WN) __attribute__((amdgpu_waves_per_eu(3, 3)))
moe_gemm_mfma128_kernel(bf16* __restrict__ out, int ld_out, const bf16* __restrict__ X, int ldx, const int* __restrict__ perm, int top,
                        const float* __restrict__ pair_w, const bf16* __restrict__ W, size_t w_expert, int ldw, const int* __restrict__ tiles,
                        const int* __restrict__ n_tiles, int N, int K, float limit, float alpha, int act, int n_slices) {
    constexpr int THREADS = 128 * WN, RSTEP = THREADS / 8, XL = MOE_BM / RSTEP, WROWS = 64 * WN, WL = WROWS / RSTEP, HALF = 32 * WN;
    constexpr int TN = GLU ? HALF : WROWS;
    __shared__ __attribute__((aligned(16))) bf16 xs[MOE_BM * MOE_LD];
    __shared__ __attribute__((aligned(16))) bf16 ws[WROWS * MOE_LD];
    __shared__ int src_row[MOE_BM];
    __shared__ float src_w[MOE_BM];
    // Workgroups go to the eight XCDs in turn, and each XCD has a second-level cache of its own: workgroup 8 a + b takes the
    // piece b * per + a of the work, so an XCD keeps a run of neighbouring pieces.  Along the pieces, MOE_BGROUP row tiles (of one
    // expert, where it has that many) take the same slice of outputs one after the other and then the next slice: the slice of W
    // comes from memory once for the group, and the group's rows of X stay in that cache while the slices pass.
    const int nt = *n_tiles, total = nt * n_slices, per = (total + 7) >> 3;
    const int piece = (int)(blockIdx.x & 7) * per + (int)(blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= per || piece >= total) return;
    const int first = piece / (MOE_BGROUP * n_slices) * MOE_BGROUP, in_group = piece % (MOE_BGROUP * n_slices);
    const int gsz = nt - first < MOE_BGROUP ? nt - first : MOE_BGROUP;
    const int tile = first + in_group % gsz;
    const int e = tiles[3 * tile], place0 = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
    const int n0 = in_group / gsz * TN, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, wm = wave / WN, wn = wave % WN;
    if (tid < MOE_BM) {
        int row = -1;
        float w = 1.0f;
        if (tid < rows) {
            if (GLU || perm != nullptr) {     // rows gathered from the tokens' rows (the plain form: only with a list of pairs)
                const int pair = perm != nullptr ? perm[place0 + tid] : place0 + tid;
                row = pair / top;
                if (pair_w != nullptr) w = pair_w[pair];
            } else {
                row = place0 + tid;
            }
        }
        src_row[tid] = row;
        src_w[tid] = w;
    }
    __syncthreads();
    const bf16* We = W + (size_t)e * w_expert;
    const int lr = tid >> 3, lc = tid & 7;        // this thread loads rows lr + RSTEP i of both tiles, 16 bytes at k chunk lc
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    uint4 xr[XL], wr[WL];
    int xrow[XL], wrow[WL];
#pragma unroll
    for (int i = 0; i < XL; ++i) xrow[i] = src_row[lr + RSTEP * i];
#pragma unroll
    for (int i = 0; i < WL; ++i) {
        const int r = lr + RSTEP * i;             // row of the W tile -> row of the expert's matrix (-1: beyond the outputs)
        const int n = GLU ? n0 + (r % HALF) : n0 + r;
        wrow[i] = n < N ? (GLU && r >= HALF ? N + n : n) : -1;
    }
    auto load = [&](int k0) {
        const int k = k0 + lc * 8;
        const bool kok = k < K;
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            uint4 v = zero;
            if (kok && xrow[i] >= 0) v = *reinterpret_cast<const uint4*>(X + (size_t)xrow[i] * ldx + k);
            xr[i] = v;
        }
#pragma unroll
        for (int i = 0; i < WL; ++i) {
            uint4 u = zero;
            if (kok && wrow[i] >= 0) u = *reinterpret_cast<const uint4*>(We + (size_t)wrow[i] * ldw + k);
            wr[i] = u;
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int i = 0; i < XL; ++i) *reinterpret_cast<uint4*>(&xs[(lr + RSTEP * i) * MOE_LD + lc * 8]) = xr[i];
#pragma unroll
        for (int i = 0; i < WL; ++i) *reinterpret_cast<uint4*>(&ws[(lr + RSTEP * i) * MOE_LD + lc * 8]) = wr[i];
    };
    f32x4 acc[4][4];
#pragma unroll
    for (int f = 0; f < 4; ++f)
#pragma unroll
        for (int g = 0; g < 4; ++g) acc[f][g] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int r16 = lane & 15, q = lane >> 4;
    // fragment f of this wave in the W tile: GLU gate tiles 0, 1 and up tiles 2, 3 of outputs 32 wn ..; else outputs 64 wn ..
    int wbase[4];
#pragma unroll
    for (int f = 0; f < 4; ++f) wbase[f] = GLU ? (f >> 1) * HALF + wn * 32 + (f & 1) * 16 : wn * 64 + f * 16;
    const int my_rows = rows - wm * 64;           // rows of this wave's half that exist
    const int groups = my_rows <= 0 ? 0 : (my_rows >= 64 ? 4 : (my_rows + 15) >> 4);
    auto compute = [&]() {
        if (groups == 4) {         // a full half: all fragments first, then sixteen products with no branch between them
#pragma unroll
            for (int ks = 0; ks < MOE_KS / 32; ++ks) {
                uint4 a[4], b[4];
#pragma unroll
                for (int f = 0; f < 4; ++f) a[f] = *reinterpret_cast<const uint4*>(&ws[(wbase[f] + r16) * MOE_LD + ks * 32 + q * 8]);
#pragma unroll
                for (int g = 0; g < 4; ++g) b[g] = *reinterpret_cast<const uint4*>(&xs[(wm * 64 + g * 16 + r16) * MOE_LD + ks * 32 + q * 8]);
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int f = 0; f < 4; ++f)
                        acc[f][g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[f]), __builtin_bit_cast(bf16x8, b[g]),
                                                                            acc[f][g], 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int ks = 0; ks < MOE_KS / 32; ++ks) {
                uint4 a[4];
#pragma unroll
                for (int f = 0; f < 4; ++f) a[f] = *reinterpret_cast<const uint4*>(&ws[(wbase[f] + r16) * MOE_LD + ks * 32 + q * 8]);
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    if (g < groups) {
                        const uint4 b = *reinterpret_cast<const uint4*>(&xs[(wm * 64 + g * 16 + r16) * MOE_LD + ks * 32 + q * 8]);
#pragma unroll
                        for (int f = 0; f < 4; ++f)
                            acc[f][g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[f]), __builtin_bit_cast(bf16x8, b),
                                                                                acc[f][g], 0, 0, 0);
                    }
                }
            }
        }
    };
    // (Tried and slower at 16 experts x 256 rows, width 4,096: loads two k-steps ahead in a second set of registers, 550 against
    // 513 us gate/up; the same with every load issued without a branch around it spilled registers.)
    load(0);
    for (int k0 = 0; k0 < K; k0 += MOE_KS) {
        __syncthreads();           // the last step's readers are done
        stage();
        __syncthreads();
        if (k0 + MOE_KS < K) load(k0 + MOE_KS);
        compute();
    }
    // lane holds rows m = 64 wm + 16 g + r16 and, of fragment f, the W rows 4 q + i
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const int m = wm * 64 + g * 16 + r16;
        if (m >= rows) continue;
        bf16* orow = out + (size_t)(place0 + m) * ld_out;
        const float sw = src_w[m];                // the pair's score: W (s x) = s (W x), taken on the float sums before the limits
#pragma unroll
        for (int f = 0; f < (GLU ? 2 : 4); ++f) {
            const int nb = GLU ? n0 + wn * 32 + f * 16 + q * 4 : n0 + wn * 64 + f * 16 + q * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (nb + i < N) {
                    float v = acc[f][g][i];
                    if (GLU) v = moe_glu(sw * v, sw * acc[f + 2][g][i], limit, alpha);
                    else if (act == 1) { v = fmaxf(v, 0.f); v *= v; }
                    orow[nb + i] = from_f32<bf16>(v);
                }
            }
        }
    }
}

// Any dtype and size, FMA in ascending k.  Block 256 threads, tile 64 rows x 64 outputs, thread (ty, tx) owns rows
// 4 ty .. 4 ty + 3 and outputs tx, tx + 16, tx + 32, tx + 48.
template <typename T, bool GLU>
__global__ void __launch_bounds__(256)
moe_gemm_plain_kernel(T* __restrict__ out, int ld_out, const T* __restrict__ X, int ldx, const int* __restrict__ perm, int top,
                      const float* __restrict__ pair_w, const T* __restrict__ W, size_t w_expert, int ldw, const int* __restrict__ tiles,
                      const int* __restrict__ n_tiles, int N, int K, float limit, float alpha, int act) {
    constexpr int WR = GLU ? 2 : 1;
    constexpr int KS = 16;
    __shared__ float xs[KS][MOE_TM + 1];
    __shared__ float ws[WR][KS][MOE_TN + 1];
    __shared__ int src_row[MOE_TM];
    __shared__ float src_w[MOE_TM];
    const int tile = blockIdx.y;
    if (tile >= *n_tiles) return;
    const int e = tiles[3 * tile], place0 = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
    const int n0 = blockIdx.x * MOE_TN, tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    if (tid < MOE_TM) {
        int row = -1;
        float w = 1.0f;
        if (tid < rows) {
            if (GLU || perm != nullptr) {     // rows gathered from the tokens' rows (the plain form: only with a list of pairs)
                const int pair = perm != nullptr ? perm[place0 + tid] : place0 + tid;
                row = pair / top;
                if (pair_w != nullptr) w = pair_w[pair];
            } else {
                row = place0 + tid;
            }
        }
        src_row[tid] = row;
        src_w[tid] = w;
    }
    __syncthreads();
    const T* We = W + (size_t)e * w_expert;
    float acc[WR][4][4];
#pragma unroll
    for (int h = 0; h < WR; ++h)
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int b = 0; b < 4; ++b) acc[h][a][b] = 0.f;
    for (int k0 = 0; k0 < K; k0 += KS) {
        for (int i = tid; i < MOE_TM * KS; i += 256) {
            const int m = i / KS, kk = i % KS, r = src_row[m];
            float v = 0.f;
            if (r >= 0 && k0 + kk < K) {
                v = to_f32(X[(size_t)r * ldx + k0 + kk]);
                if (GLU) v = to_f32(from_f32<T>(v * src_w[m]));
            }
            xs[kk][m] = v;
        }
        for (int i = tid; i < WR * MOE_TN * KS; i += 256) {
            const int h = i / (MOE_TN * KS), n = (i / KS) % MOE_TN, kk = i % KS;
            ws[h][kk][n] = (n0 + n < N && k0 + kk < K) ? to_f32(We[(size_t)(h * N + n0 + n) * ldw + k0 + kk]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
            float xv[4];
#pragma unroll
            for (int a = 0; a < 4; ++a) xv[a] = xs[kk][ty * 4 + a];
#pragma unroll
            for (int h = 0; h < WR; ++h)
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const float wv = ws[h][kk][tx + 16 * b];
#pragma unroll
                    for (int a = 0; a < 4; ++a) acc[h][a][b] = fmaf(xv[a], wv, acc[h][a][b]);
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        const int m = ty * 4 + a;
        if (m >= rows) continue;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int n = n0 + tx + 16 * b;
            if (n < N) {
                float v = acc[0][a][b];
                if (GLU) v = moe_glu(v, acc[WR - 1][a][b], limit, alpha);
                else if (act == 1) { v = fmaxf(v, 0.f); v *= v; }
                out[(size_t)(place0 + m) * ld_out + n] = from_f32<T>(v);
            }
        }
    }
}

extern "C" int ilm_moe_gemm(void* out, int ld_out, const void* X, int ldx, const void* perm, int top, const void* pair_w, const void* W,
                            long w_expert, int ldw, const void* tiles, const void* n_tiles, int max_tiles, int N, int K, int glu,
                            float limit, float alpha, int act, int dtype, int force_plain, int tile_rows, int wide_mode, hipStream_t stream) {
    ILM_REQUIRE(act == 0 || (act == 1 && !glu), "moe_gemm: activation %d (0: none, 1: the square of relu, in the plain form)", act);
    ILM_REQUIRE(tile_rows == MOE_TM || tile_rows == MOE_BM, "moe_gemm: tiles of %d rows (%d or %d)", tile_rows, MOE_TM, MOE_BM);
    ILM_REQUIRE(max_tiles > 0 && max_tiles <= 65535 && N > 0 && K > 0 && top > 0, "moe_gemm: bad sizes (tiles %d, N %d, K %d)", max_tiles, N, K);
    ILM_REQUIRE(ld_out >= N && ldx >= K && ldw >= K, "moe_gemm: rows shorter than their products");
    dim3 grid((N + MOE_TN - 1) / MOE_TN, max_tiles);
#define MOE_ARGS(T__) (T__*)out, ld_out, (const T__*)X, ldx, (const int*)perm, top, (const float*)pair_w, (const T__*)W, (size_t)w_expert, ldw, \
                      (const int*)tiles, (const int*)n_tiles, N, K, limit, alpha, act
    const bool aligned = K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0 && w_expert % 8 == 0 && ((uintptr_t)X % 16) == 0 && ((uintptr_t)W % 16) == 0;
    if (dtype == ILM_DTYPE_BF16 && aligned && !force_plain && tile_rows == MOE_BM) {
        // 256 rows of W a tile on demand (wide_mode 1) where the outputs fill one: a third fewer bytes a product from the caches, and
        // slower all the same at 16 experts x 256 rows, width 4,096 (622 against 545 us gate/up, 345 against 308 us down)
        const int wide_slices = glu ? (N + 127) / 128 : (N + 255) / 256;
        const bool wide = (glu ? N >= 128 : N >= 256) && (wide_mode & 1);
        const int n_slices = wide ? wide_slices : (glu ? (N + 63) / 64 : (N + 127) / 128);
        ILM_REQUIRE((long)max_tiles * n_slices < (1L << 30), "moe_gemm: %d tiles of %d slices are too many", max_tiles, n_slices);
        const int big = (max_tiles * n_slices + 7) / 8 * 8;      // (a multiple of 8, so every XCD's run has a workgroup for each piece)
        if (glu && wide) moe_gemm_mfma128_kernel<true, 4><<<big, 512, 0, stream>>>(MOE_ARGS(bf16), n_slices);
        else if (glu) moe_gemm_mfma128_kernel<true, 2><<<big, 256, 0, stream>>>(MOE_ARGS(bf16), n_slices);
        else if (wide) moe_gemm_mfma128_kernel<false, 4><<<big, 512, 0, stream>>>(MOE_ARGS(bf16), n_slices);
        else moe_gemm_mfma128_kernel<false, 2><<<big, 256, 0, stream>>>(MOE_ARGS(bf16), n_slices);
    } else if (tile_rows != MOE_TM) {
        ILM_REQUIRE(false, "moe_gemm: tiles of %d rows are the bfloat16 matrix-core kernel's alone", tile_rows);
    } else if (dtype == ILM_DTYPE_BF16 && aligned && !force_plain) {
        if (glu) moe_gemm_mfma_kernel<true><<<grid, 256, 0, stream>>>(MOE_ARGS(bf16));
        // (on demand, and only where an expert's matrix is large.  Measured, 64 tokens x 2 of 8 experts, with one set of load
        // registers: 8192 x 4096 a matrix 175 -> 149 us, 4096 x 8192 204 -> 193; with two sets 132 against 135 and 129 against 138)
        else if ((wide_mode & 2) && N >= 2 * MOE_TN && (long)N * K >= (1L << 23))
            moe_gemm_mfma_kernel<false, true><<<dim3((N + 2 * MOE_TN - 1) / (2 * MOE_TN), max_tiles), 256, 0, stream>>>(MOE_ARGS(bf16));
        else moe_gemm_mfma_kernel<false><<<grid, 256, 0, stream>>>(MOE_ARGS(bf16));
    } else if (dtype == ILM_DTYPE_BF16) {
        if (glu) moe_gemm_plain_kernel<bf16, true><<<grid, 256, 0, stream>>>(MOE_ARGS(bf16));
        else moe_gemm_plain_kernel<bf16, false><<<grid, 256, 0, stream>>>(MOE_ARGS(bf16));
    } else if (dtype == ILM_DTYPE_F32) {
        if (glu) moe_gemm_plain_kernel<float, true><<<grid, 256, 0, stream>>>(MOE_ARGS(float));
        else moe_gemm_plain_kernel<float, false><<<grid, 256, 0, stream>>>(MOE_ARGS(float));
    } else {
        ILM_REQUIRE(false, "moe_gemm: unknown dtype %d", dtype);
    }
#undef MOE_ARGS
    ILM_LAUNCH_CHECK("moe_gemm");
    return 0;
}

// ---- the sum over a token's experts --------------------------------------------------------------------------------
template <typename T>
__global__ void moe_combine_kernel(T* __restrict__ y, const T* __restrict__ pair_out, const int* __restrict__ inv, int top,
                                   const T* __restrict__ shared, const float* __restrict__ sg, int sg_stride, int H, int ld_pair,
                                   const float* __restrict__ pair_w) {
    const int t = blockIdx.x;
    const float gate = sg != nullptr ? moe_sigmoid(sg[(size_t)t * sg_stride]) : 1.0f;
    for (int j = threadIdx.x; j < H; j += blockDim.x) {
        float v = 0.f;
        for (int s = 0; s < top; ++s) {
            const float o = to_f32(pair_out[(size_t)inv[(size_t)t * top + s] * ld_pair + j]);
            v = pair_w != nullptr ? fmaf(pair_w[(size_t)t * top + s], o, v) : v + o;
        }
        if (shared != nullptr) v = fmaf(to_f32(shared[(size_t)t * H + j]), gate, v);
        y[(size_t)t * H + j] = from_f32<T>(v);
    }
}

extern "C" int ilm_moe_combine(void* y, const void* pair_out, const void* inv, int top, const void* shared, const void* sg, int sg_stride,
                               int T_, int H, int ld_pair, const void* pair_w, int dtype, hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && H > 0 && top > 0 && ld_pair >= H, "moe_combine: bad sizes");
    if (dtype == ILM_DTYPE_F32)
        moe_combine_kernel<float><<<T_, 256, 0, stream>>>((float*)y, (const float*)pair_out, (const int*)inv, top, (const float*)shared,
                                                          (const float*)sg, sg_stride, H, ld_pair, (const float*)pair_w);
    else if (dtype == ILM_DTYPE_BF16)
        moe_combine_kernel<bf16><<<T_, 256, 0, stream>>>((bf16*)y, (const bf16*)pair_out, (const int*)inv, top, (const bf16*)shared,
                                                         (const float*)sg, sg_stride, H, ld_pair, (const float*)pair_w);
    else
        ILM_REQUIRE(false, "moe_combine: unknown dtype %d", dtype);
    ILM_LAUNCH_CHECK("moe_combine");
    return 0;
}

// ---- the activation alone, on fused [gate | up] rows ---------------------------------------------------------------
template <typename T>
__global__ void glu_clamp_kernel(T* __restrict__ out, const T* __restrict__ gu, int I, int gu_stride, float limit, float alpha, long total) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const long t = i / I;
    const int j = (int)(i % I);
    const T* row = gu + (size_t)t * gu_stride;
    out[(size_t)t * I + j] = from_f32<T>(moe_glu(to_f32(row[j]), to_f32(row[I + j]), limit, alpha));
}

extern "C" int ilm_glu_clamp(void* out, const void* gu, int T_, int I, int gu_stride, float limit, float alpha, int dtype, hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && I > 0 && gu_stride >= 2 * I, "glu_clamp: bad sizes");
    const long total = (long)T_ * I;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (dtype == ILM_DTYPE_F32) glu_clamp_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, (const float*)gu, I, gu_stride, limit, alpha, total);
    else if (dtype == ILM_DTYPE_BF16) glu_clamp_kernel<bf16><<<blocks, 256, 0, stream>>>((bf16*)out, (const bf16*)gu, I, gu_stride, limit, alpha, total);
    else ILM_REQUIRE(false, "glu_clamp: unknown dtype %d", dtype);
    ILM_LAUNCH_CHECK("glu_clamp");
    return 0;
}
