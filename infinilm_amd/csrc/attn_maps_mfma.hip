// Differential attention on the matrix cores (bfloat16), a head's two maps in one pass.
//
//   a_m = softmax(scale q_hm K_gm^T over the window) V_g,  m = 0, 1        (K_gm: entries m dim .. of the cached key rows)
//   o = a_0 - lambda a_1,  lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff
//   out = o / sqrt(mean(o^2 over vdim) + eps) * out_scale
//
// A workgroup = one item (a tile of up to 16 consecutive tokens of a request, or a single token) x four heads of one
// key/value head, a wave a head.  Keys go by in tiles of 32 aligned to the absolute key index; the K [key][d] and V [d][key]
// tile of the group passes through LDS once for the four heads and both maps, the next tile's loads in flight meanwhile.
// Per head, map and tile (v_mfma_f32_16x16x32_bf16):
//   S^T [keys x 16 tokens] = K_m q_m^T        dim / 32 k-steps over the map's part of the key rows
//   running maximum, sum and weights per token, float
//   O_m^T [d x 16 tokens] += V^T P_m^T        the weights as two bfloat16 terms (the rounded weight and the rest), so
//                                              16 bits of each float weight count; both maps read the same V fragments
// and at the end the two results are combined, normed and scaled in the registers they lie in.  Scores, maxima,
// exponentials, sums, lambda and the norm are float.  A token's result depends on its position and its request's cache
// alone: keys outside its window weigh exactly zero and leave its running maximum alone.
//
// Sizes: dim and the cache's head size d multiples of 32, d <= 128, pages of a multiple of 32.  Decoded tokens over long
// windows are better served by the chunked form of ilm_attn_headmix_mfma (keys over more workgroups); this kernel walks an
// item's keys in one workgroup.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 am_bf16x8;
typedef __attribute__((ext_vector_type(4))) float am_f32x4;

#define AMX_NEG (-1.0e30f)
#define AMX_TK 32

__device__ __forceinline__ am_f32x4 am_mfma(uint4 a, uint4 b, am_f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(am_bf16x8, a), __builtin_bit_cast(am_bf16x8, b), c, 0, 0, 0);
}

__device__ __forceinline__ uint32_t am_pack(float lo, float hi) {
    return (uint32_t)from_f32<bf16>(lo).bits | ((uint32_t)from_f32<bf16>(hi).bits << 16);
}

template <int D32, int DQ32, typename TW>
__global__ void __launch_bounds__(256)
attn_maps_mfma_kernel(bf16* __restrict__ out, const bf16* __restrict__ q, const bf16* __restrict__ kc, const bf16* __restrict__ vc,
                      const int* __restrict__ block_tables, const int* __restrict__ seg, const int* __restrict__ pos,
                      const int* __restrict__ tiles, int n_tiles, const int* __restrict__ singles, int H, int G, int vdim, int page,
                      int max_blocks, int out_stride, float scale_log2e, int window, const int* __restrict__ seg_offsets,
                      const TW* __restrict__ lq1, const TW* __restrict__ lk1, const TW* __restrict__ lq2, const TW* __restrict__ lk2,
                      float diff, float norm_eps, float out_scale) {
    constexpr int D = D32 * 32, DIM = DQ32 * 32, TK = AMX_TK, KROW = D + 8, VROW = TK + 8, NS = TK / 16, NP = TK / 32;
    __shared__ __attribute__((aligned(16))) bf16 Ks[TK * KROW];        // [key][d]
    __shared__ __attribute__((aligned(16))) bf16 Vs[D * VROW];         // [d][key]
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 15, g4 = lane >> 4, wave = tid >> 6;
    int t0, ntok;
    if ((int)blockIdx.x < n_tiles) {
        t0 = tiles[2 * blockIdx.x];
        ntok = tiles[2 * blockIdx.x + 1];
        // the step's lists hold tiles of up to 8 tokens, cut from each request's first row on: the even tiles of a request take
        // their successors' tokens along (16 columns), the odd ones leave
        if (seg_offsets != nullptr && ntok > 0) {
            const int sg = seg[t0], first = seg_offsets[sg], end = seg_offsets[sg + 1];
            if (((t0 - first) >> 3) & 1) return;
            ntok = min(16, end - t0);
        }
    } else {
        const int i = blockIdx.x - n_tiles;
        t0 = singles != nullptr ? singles[i] : i;
        ntok = t0 >= 0 ? 1 : 0;
    }
    if (ntok <= 0) return;                                       // an entry that fills up a recorded step's lists
    const int per = H / G, passes = (per + 3) / 4;
    const int g = blockIdx.y / passes, in_group = (blockIdx.y % passes) * 4 + wave;
    const bool head_ok = in_group < per;                         // (uniform over the wave; idle waves still load tiles and meet the barriers)
    const int h = g * per + (head_ok ? in_group : 0);
    const int p_first = pos[t0], p_last = p_first + ntok - 1;
    const int lo_first = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
    const int* bt = block_tables + (size_t)seg[t0] * max_blocks;
    const bool tok_ok = r < ntok;
    const int tok = t0 + (tok_ok ? r : 0);
    const int p_tok = p_first + (tok_ok ? r : 0);
    const int lo_tok = (window > 0 && p_tok - window + 1 > 0) ? p_tok - window + 1 : 0;
    // lambda: every wave forms it for itself (2 x dim multiply-adds)
    float la = 0.f, lb = 0.f;
    for (int e = lane; e < DIM; e += 64) {
        la = fmaf(to_f32(lq1[e]), to_f32(lk1[e]), la);
        lb = fmaf(to_f32(lq2[e]), to_f32(lk2[e]), lb);
    }
    const float lambda = expf(wave_sum(la)) - expf(wave_sum(lb)) + diff;
    // this wave's head: the two maps' queries of this lane's token
    uint4 qf[2][DQ32];
    am_f32x4 O[2][2 * D32];
    float m_run[2], l_run[2];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
        const bf16* qrow = q + (((size_t)tok * H + h) * 2 + m) * DIM;
#pragma unroll
        for (int ks = 0; ks < DQ32; ++ks) qf[m][ks] = *reinterpret_cast<const uint4*>(qrow + ks * 32 + g4 * 8);
#pragma unroll
        for (int b = 0; b < 2 * D32; ++b) O[m][b] = am_f32x4{0.f, 0.f, 0.f, 0.f};
        m_run[m] = AMX_NEG;
        l_run[m] = 0.f;
    }
    constexpr int KPIECES = TK * (D / 8), VPIECES = D * (TK / 8);
    constexpr int KPER = (KPIECES + 255) / 256, VPER = (VPIECES + 255) / 256;
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
    uint4 kreg[KPER], vreg[VPER];
    auto fetch = [&](int kb) {
        const int pg = bt[kb / page];                            // (a tile lies on one page: the page size is a multiple of 32)
        const int off = kb % page;                               // pg < 0: a page the window has passed; its keys weigh nothing
#pragma unroll
        for (int i = 0; i < KPER; ++i) {
            const int pc = tid + i * 256;
            const int key = pc / (D / 8), piece = pc % (D / 8);
            kreg[i] = zero4;
            if (pc < KPIECES && pg >= 0) kreg[i] = *reinterpret_cast<const uint4*>(kc + (((size_t)pg * G + g) * page + off + key) * D + piece * 8);
        }
#pragma unroll
        for (int i = 0; i < VPER; ++i) {
            const int pc = tid + i * 256;
            const int row = pc / (TK / 8), piece = pc % (TK / 8);
            vreg[i] = zero4;
            if (pc < VPIECES && pg >= 0) vreg[i] = *reinterpret_cast<const uint4*>(vc + (((size_t)pg * G + g) * D + row) * page + off + piece * 8);
        }
    };
    const int kb_begin = lo_first & ~(TK - 1), kb_end = p_last;
    if (kb_begin <= kb_end) fetch(kb_begin);
    for (int kb = kb_begin; kb <= kb_end; kb += TK) {
        __syncthreads();                                         // the tile before this one has been read by every wave
#pragma unroll
        for (int i = 0; i < KPER; ++i) {
            const int pc = tid + i * 256;
            const int key = pc / (D / 8), piece = pc % (D / 8);
            if (pc < KPIECES) *reinterpret_cast<uint4*>(Ks + key * KROW + piece * 8) = kreg[i];
        }
#pragma unroll
        for (int i = 0; i < VPER; ++i) {
            const int pc = tid + i * 256;
            const int row = pc / (TK / 8), piece = pc % (TK / 8);
            if (pc < VPIECES) *reinterpret_cast<uint4*>(Vs + row * VROW + piece * 8) = vreg[i];
        }
        __syncthreads();
        if (kb + TK <= kb_end) fetch(kb + TK);
        if (!head_ok) continue;
        // the weights of both maps first, then the value products: a V fragment read from LDS serves both maps
        uint4 pb[2][NP], pb_lo[2][NP];
        float corr[2];
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            am_f32x4 S[NS];
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                S[s] = am_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < DQ32; ++ks) {
                    const uint4 a = *reinterpret_cast<const uint4*>(Ks + (s * 16 + r) * KROW + m * DIM + ks * 32 + g4 * 8);
                    S[s] = am_mfma(a, qf[m][ks], S[s]);
                }
            }
            // this lane: token r, keys kb + 16 s + 4 g4 + j
            float sc[4 * NS];
            float mx = AMX_NEG;
#pragma unroll
            for (int s = 0; s < NS; ++s)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int key = kb + s * 16 + g4 * 4 + j;
                    const bool seen = tok_ok && key >= lo_tok && key <= p_tok;
                    sc[s * 4 + j] = seen ? S[s][j] * scale_log2e : AMX_NEG;
                    mx = fmaxf(mx, sc[s * 4 + j]);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m_run[m], mx);
            corr[m] = __builtin_amdgcn_exp2f(m_run[m] - m_new);
            float pw[4 * NS], sum = 0.f;
#pragma unroll
            for (int j = 0; j < 4 * NS; ++j) {
                pw[j] = sc[j] > 0.5f * AMX_NEG ? __builtin_amdgcn_exp2f(sc[j] - m_new) : 0.f;
                sum += pw[j];
            }
            l_run[m] = l_run[m] * corr[m] + sum;                 // (this lane's share; the four lanes of a token are summed at the end)
            m_run[m] = m_new;
#pragma unroll
            for (int u = 0; u < NP; ++u) {
                float pl[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) pl[j] = pw[8 * u + j] - to_f32(from_f32<bf16>(pw[8 * u + j]));
                pb[m][u] = make_uint4(am_pack(pw[8 * u], pw[8 * u + 1]), am_pack(pw[8 * u + 2], pw[8 * u + 3]),
                                      am_pack(pw[8 * u + 4], pw[8 * u + 5]), am_pack(pw[8 * u + 6], pw[8 * u + 7]));
                pb_lo[m][u] = make_uint4(am_pack(pl[0], pl[1]), am_pack(pl[2], pl[3]), am_pack(pl[4], pl[5]), am_pack(pl[6], pl[7]));
            }
        }
#pragma unroll
        for (int b = 0; b < 2 * D32; ++b) {
            const bf16* vrow = Vs + (b * 16 + r) * VROW;
            am_f32x4 o0 = O[0][b], o1 = O[1][b];
            o0[0] *= corr[0]; o0[1] *= corr[0]; o0[2] *= corr[0]; o0[3] *= corr[0];
            o1[0] *= corr[1]; o1[1] *= corr[1]; o1[2] *= corr[1]; o1[3] *= corr[1];
#pragma unroll
            for (int u = 0; u < NP; ++u) {
                const uint2 v0 = *reinterpret_cast<const uint2*>(vrow + 32 * u + g4 * 4);          // keys 32 u + 4 g4 .. + 3
                const uint2 v1 = *reinterpret_cast<const uint2*>(vrow + 32 * u + 16 + g4 * 4);     // keys 32 u + 16 + 4 g4 .. + 3
                const uint4 va = make_uint4(v0.x, v0.y, v1.x, v1.y);
                o0 = am_mfma(va, pb_lo[0][u], am_mfma(va, pb[0][u], o0));
                o1 = am_mfma(va, pb_lo[1][u], am_mfma(va, pb[1][u], o1));
            }
            O[0][b] = o0;
            O[1][b] = o1;
        }
    }
    if (!head_ok) return;
    float inv[2];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
        float l = l_run[m];
        l += __shfl_xor(l, 16, 64);
        l += __shfl_xor(l, 32, 64);
        inv[m] = 1.0f / l;
    }
    // o = a_0 - lambda a_1 where the results lie (this lane: token r, value entries 16 b + 4 g4 + j), then the root mean square
    // over the token's vdim entries, which four lanes hold
    const float w1 = lambda * inv[1];
    float ss = 0.f;
#pragma unroll
    for (int b = 0; b < 2 * D32; ++b)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float o = O[0][b][j] * inv[0] - w1 * O[1][b][j];
            O[0][b][j] = o;
            if (b * 16 + g4 * 4 + j < vdim) ss = fmaf(o, o, ss);
        }
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    const float f = norm_eps >= 0.f ? out_scale / sqrtf(ss / (float)vdim + norm_eps) : out_scale;
    if (tok_ok) {
        bf16* orow = out + (size_t)tok * out_stride + (size_t)h * vdim;
#pragma unroll
        for (int b = 0; b < 2 * D32; ++b)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int e = b * 16 + g4 * 4 + j;
                if (e < vdim) orow[e] = from_f32<bf16>(O[0][b][j] * f);
            }
    }
}

extern "C" int ilm_attn_maps_mfma_ok(int H, int G, int dim, int vdim, int d, int page) {
    return H > 0 && G > 0 && H % G == 0 && dim % 32 == 0 && dim >= 32 && d % 32 == 0 && d <= 128 && 2 * dim <= d && vdim > 0 && vdim <= d &&
           page % 32 == 0;
}

// q [T, H, 2, dim] dense; tiles [n_tiles, 2] = (first row, count <= 8) and n_singles single rows (`singles` null: rows
// 0 .. n_singles - 1; an entry -1 or a count 0 names nothing); seg_offsets (may be null): the first row of every request of the
// step and the end of the last, with which tiles cut 8 by 8 from a request's first row are served two at a time; out [T, H vdim]
extern "C" int ilm_attn_maps_mfma(void* out, const void* q, const void* kc, const void* vc, const void* block_tables, const void* seg,
                                  const void* pos, const void* tiles, int n_tiles, const void* singles, int n_singles, int H, int G,
                                  int dim, int vdim, int d, int page, int max_blocks, int out_stride, float scale, int window,
                                  const void* seg_offsets, const void* lq1, const void* lk1, const void* lq2, const void* lk2, float diff,
                                  float norm_eps, float out_scale, int w_dt, hipStream_t stream) {
    ILM_REQUIRE(n_tiles >= 0 && n_singles >= 0 && n_tiles + n_singles > 0 && max_blocks > 0, "attn_maps_mfma: bad sizes");
    ILM_REQUIRE(ilm_attn_maps_mfma_ok(H, G, dim, vdim, d, page), "attn_maps_mfma: %d heads in %d groups, maps of %d, values of %d, cache heads of %d, pages of %d",
                H, G, dim, vdim, d, page);
    ILM_REQUIRE(((uintptr_t)q & 15) == 0 && ((uintptr_t)kc & 15) == 0 && ((uintptr_t)vc & 15) == 0 && out_stride >= H * vdim,
                "attn_maps_mfma: rows must be 16-byte aligned");
    ILM_REQUIRE(lq1 && lk1 && lq2 && lk2 && window >= 0, "attn_maps_mfma: the four vectors of the maps' weight are needed");
    const float scale_log2e = scale * 1.4426950408889634f;
    const int per = H / G;
    dim3 grid(n_tiles + n_singles, G * ((per + 3) / 4));
#define AMX_LAUNCH(D32_, DQ32_, TW_)                                                                                          \
    attn_maps_mfma_kernel<D32_, DQ32_, TW_><<<grid, 256, 0, stream>>>(                                                        \
        (bf16*)out, (const bf16*)q, (const bf16*)kc, (const bf16*)vc, (const int*)block_tables, (const int*)seg, (const int*)pos, \
        (const int*)tiles, n_tiles, (const int*)singles, H, G, vdim, page, max_blocks, out_stride, scale_log2e, window,       \
        (const int*)seg_offsets, (const TW_*)lq1, (const TW_*)lk1, (const TW_*)lq2, (const TW_*)lk2, diff, norm_eps, out_scale)
#define AMX_BY_DT(D32_, DQ32_)                                       \
    if (w_dt == ILM_DTYPE_BF16) AMX_LAUNCH(D32_, DQ32_, bf16);       \
    else if (w_dt == ILM_DTYPE_F32) AMX_LAUNCH(D32_, DQ32_, float);  \
    else ILM_REQUIRE(false, "attn_maps_mfma: dtype %d", w_dt);
    const int d32 = d / 32, dq32 = dim / 32;
    if (d32 == 2 && dq32 == 1) { AMX_BY_DT(2, 1) }
    else if (d32 == 3 && dq32 == 1) { AMX_BY_DT(3, 1) }
    else if (d32 == 4 && dq32 == 1) { AMX_BY_DT(4, 1) }
    else if (d32 == 4 && dq32 == 2) { AMX_BY_DT(4, 2) }
    else ILM_REQUIRE(false, "attn_maps_mfma: cache heads of %d with maps of %d", d, dim);
#undef AMX_BY_DT
#undef AMX_LAUNCH
    ILM_LAUNCH_CHECK("attn_maps_mfma");
    return 0;
}
