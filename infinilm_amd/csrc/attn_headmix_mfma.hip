// Attention with scores mixed over the heads, on the matrix cores (bfloat16).
//
// The mixing is carried into the queries: with s_h(j) = sum_g M[h, g] scale q_g . k_kv(g),j and C key/value groups,
//   s_h(j) = scale sum_c q'_{h,c} . k_{c,j},    q'_{h,c} = sum_{g in group c} M[h, g] q_g,
// so head h asks with a query of C d entries against the key row [k_0,j | ... | k_{C-1},j] of all groups, and takes its
// values from its own group.  `ilm_headmix_queries` forms q' (float sums, bfloat16 result: a query like any other
// operand of the score product); `ilm_attn_headmix_mfma` is then a flash attention over the window with one more term
// exp(sink_h) in the denominator (and, with `keep_first`, over the sequence's first keys as well).  Cost of the score product: C times that of unmixed heads, and no exchange of scores
// between heads; for many groups the plain kernel's explicit mixing does less work.
//
// A workgroup = one item (a tile of up to 16 consecutive tokens of a request, or a single token) x one pass of 4 HPW
// heads; its 4 waves take HPW heads each (for single tokens, where the groups allow it, 16 heads each: the heads are then
// the products' columns in place of the tokens).  Keys go by in tiles of 32 aligned to the absolute key index; K [group][key][d]
// and V [group][d][key] of a tile pass through LDS once for all heads of the pass.  Per head and tile:
//   S^T [keys x 16 tokens] = K q'^T           (v_mfma_f32_16x16x32_bf16: A = K rows, B = q' rows; lane (r, g4) gets
//                                              keys 4 g4 .. 4 g4 + 3 of each 16-key half for token r)
//   running maximum, sum and weights per token (a token's keys lie in 4 lanes x 8 registers)
//   O^T [d x 16 tokens] += V^T P^T            (A = V rows [d][key], B = the weights as they lie in the registers: the k index
//                                              of this product is a fixed permutation of the keys, the same for A and B)
// Scores, maxima, exponentials and sums are float; the weights enter the second product as two bfloat16 terms (hi + lo).
// Without a mixing matrix and with one group the mixed queries are the queries themselves: the kernel then is a plain flash
// attention whose weights stay float, for mixers that want them so.
// A token's result depends on its position and its request's cache alone: keys outside its window weigh exactly zero
// and leave its running maximum alone, whatever other tokens share the tile.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 hx_bf16x8;
typedef __attribute__((ext_vector_type(4))) float hx_f32x4;

#define HX_NEG (-1.0e30f)

__device__ __forceinline__ hx_f32x4 hx_mfma(uint4 a, uint4 b, hx_f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(hx_bf16x8, a), __builtin_bit_cast(hx_bf16x8, b), c, 0, 0, 0);
}

__device__ __forceinline__ uint32_t hx_pack(float lo, float hi) {
    return (uint32_t)from_f32<bf16>(lo).bits | ((uint32_t)from_f32<bf16>(hi).bits << 16);
}

// ------------------------------------------------------------------------------------------
// q' [T, nh, C, d] from q rows (head g at [g d, (g + 1) d)) and M [nh, nh] (null: the identity)
// ------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
headmix_queries_rows_kernel(bf16* __restrict__ qx, const bf16* __restrict__ q, const float* __restrict__ mix, int nh, int nkv, int d,
                       int q_stride) {
    extern __shared__ float qs[];
    const int t = blockIdx.x, per = nh / nkv;
    const bf16* row = q + (size_t)t * q_stride;
    for (int i = threadIdx.x; i < nh * d; i += 256) qs[i] = to_f32(row[i]);
    __syncthreads();
    bf16* dst = qx + (size_t)t * nh * nkv * d;
    for (int idx = threadIdx.x; idx < nh * nkv * d; idx += 256) {
        const int e = idx % d, c = (idx / d) % nkv, h = idx / (d * nkv);
        float a = 0.f;
        for (int g = c * per; g < (c + 1) * per; ++g) {
            const float m = mix != nullptr ? mix[h * nh + g] : (g == h ? 1.f : 0.f);
            a = fmaf(m, qs[g * d + e], a);
        }
        dst[idx] = from_f32<bf16>(a);
    }
}

__global__ void __launch_bounds__(256)
headmix_queries_kernel(bf16* __restrict__ qx, const bf16* __restrict__ q, const float* __restrict__ mix, int nh, int nkv, int d,
                       int q_stride) {
    // a block a (token, head h): its C d entries, each a sum over the heads of one group
    const int t = blockIdx.x, h = blockIdx.y, per = nh / nkv;
    const bf16* row = q + (size_t)t * q_stride;
    bf16* dst = qx + ((size_t)t * nh + h) * nkv * d;
    for (int idx = threadIdx.x; idx < nkv * d; idx += 256) {
        const int e = idx % d, c = idx / d;
        float a = 0.f;
        for (int g = c * per; g < (c + 1) * per; ++g) {
            const float m = mix != nullptr ? mix[h * nh + g] : (g == h ? 1.f : 0.f);
            a = fmaf(m, to_f32(row[g * d + e]), a);
        }
        dst[idx] = from_f32<bf16>(a);
    }
}

// few rows (decoded tokens): a block a (token, head); many: a block a token with its query heads in LDS
extern "C" int ilm_headmix_queries(void* qx, const void* q, const void* mix, int T_, int nh, int nkv, int d, int q_stride,
                                   hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && nh > 0 && nh <= 65535 && nkv > 0 && nh % nkv == 0 && d > 0, "headmix_queries: bad sizes");
    if (T_ >= 256 && (size_t)nh * d * sizeof(float) <= 64 * 1024)
        headmix_queries_rows_kernel<<<T_, 256, (size_t)nh * d * sizeof(float), stream>>>((bf16*)qx, (const bf16*)q, (const float*)mix, nh,
                                                                                       nkv, d, q_stride);
    else
        headmix_queries_kernel<<<dim3(T_, nh), 256, 0, stream>>>((bf16*)qx, (const bf16*)q, (const float*)mix, nh, nkv, d, q_stride);
    ILM_LAUNCH_CHECK("headmix_queries");
    return 0;
}

// ------------------------------------------------------------------------------------------
// TK: keys a tile (32; tiles of 64 halve the rounds of loads and barriers and measured slower: 437 against 374 us a
// prompt step at 32 heads of 128, more LDS a workgroup and fewer workgroups a unit)
// HC (single tokens; one key/value group, or groups of a multiple of 16 heads): the 16 columns of the products are 16 heads of one token instead
// of 16 tokens of one head (q' of head r in lane r; a wave takes 16 heads, a workgroup 64): a decoded token's keys are then
// read once for 64 heads instead of once a head.  HPW is 1.
template <int D32, int NC, int HPW, int TK, bool HC = false>
__global__ void __launch_bounds__(256)
attn_headmix_mfma_kernel(bf16* __restrict__ out, const bf16* __restrict__ qx, const bf16* __restrict__ kc, const bf16* __restrict__ vc,
                         const int* __restrict__ block_tables, const int* __restrict__ seg, const int* __restrict__ pos,
                         const int* __restrict__ tiles, int n_tiles, const int* __restrict__ singles,
                         const float* __restrict__ sink, int nh, int page, int max_blocks, int out_stride, float scale_log2e,
                         int window, float* __restrict__ ws, int chunk_keys, const int* __restrict__ seg_offsets, int keep_first,
                         int out_f32) {
    constexpr int D = D32 * 32, KROW = D + 8, VROW = TK + 8, NS = TK / 16, NP = TK / 32;
    extern __shared__ __attribute__((aligned(16))) unsigned char hx_smem[];
    bf16* Ks = reinterpret_cast<bf16*>(hx_smem);                 // [NC][32][KROW]
    bf16* Vs = Ks + NC * TK * KROW;                              // [NC][D][VROW]
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 15, g4 = lane >> 4, wave = tid >> 6;
    int t0, ntok;
    if ((int)blockIdx.x < n_tiles) {
        t0 = tiles[2 * blockIdx.x];
        ntok = tiles[2 * blockIdx.x + 1];
        // The step's lists hold tiles of up to 8 tokens, cut from each request's first row on.  With the requests' first
        // rows at hand two neighbours make one tile of 16 (all the products' columns): the even tiles of a request take
        // their successors' tokens along, the odd ones leave.
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
    const int p_first = pos[t0], p_last = p_first + ntok - 1;
    const int lo_first = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
    const int* bt = block_tables + (size_t)seg[t0] * max_blocks;
    const int per = nh / NC;
    // this lane's token (column r of the products)
    const bool tok_ok = HC || r < ntok;
    const int tok = t0 + ((tok_ok && !HC) ? r : 0);
    const int p_tok = p_first + ((tok_ok && !HC) ? r : 0);
    const int lo_tok = (window > 0 && p_tok - window + 1 > 0) ? p_tok - window + 1 : 0;
    // this wave's heads and their queries
    int head[HPW];
    bool head_ok[HPW], lane_ok[HPW];     // lane_ok: this lane's column holds a head (HC with fewer heads than columns)
    uint4 qf[HPW][NC][D32];
    hx_f32x4 O[HPW][2 * D32];
    float m_run[HPW], l_run[HPW];
#pragma unroll
    for (int i = 0; i < HPW; ++i) {
        const int h = HC ? (blockIdx.y * 4 + wave) * 16 + r : (blockIdx.y * 4 + wave) * HPW + i;
        head_ok[i] = HC ? (blockIdx.y * 4 + wave) * 16 < nh : h < nh;     // (uniform over the wave)
        lane_ok[i] = h < nh;
        head[i] = h < nh ? h : nh - 1;
        const bf16* qrow = qx + ((size_t)tok * nh + head[i]) * NC * D;
#pragma unroll
        for (int c = 0; c < NC; ++c)
#pragma unroll
            for (int ks = 0; ks < D32; ++ks) qf[i][c][ks] = *reinterpret_cast<const uint4*>(qrow + c * D + ks * 32 + g4 * 8);
#pragma unroll
        for (int b = 0; b < 2 * D32; ++b) O[i][b] = hx_f32x4{0.f, 0.f, 0.f, 0.f};
        m_run[i] = HX_NEG;
        l_run[i] = 0.f;
    }
    constexpr int KPIECES = NC * TK * (D / 8), VPIECES = NC * D * (TK / 8);
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
    // chunk_keys > 0 (single tokens over long windows): this workgroup takes the keys of chunk blockIdx.z, counted from the
    // first tile the token sees, and leaves a partial result (maximum, sum, unnormalised output) for the merge kernel
    int kb_begin = lo_first & ~(TK - 1), kb_end = p_last;
    if (chunk_keys > 0) {
        kb_begin += blockIdx.z * chunk_keys;
        kb_end = min(p_last, kb_begin + chunk_keys - 1);
    }
    // A tile is on its way from the cache into registers while the tile before it is multiplied: a workgroup's tiles are a
    // chain (load, barrier, multiply), and with one head a wave the chain's length, not the chip's throughput, sets the time
    // of a long request's last tiles.
    constexpr int KPER = (KPIECES + 255) / 256, VPER = (VPIECES + 255) / 256;
    uint4 kreg[KPER], vreg[VPER];
    auto fetch = [&](int kb) {
        const int pg = bt[kb / page];                            // (a tile lies on one page: the page size is a multiple of 32)
        const int off = kb % page;                               // pg < 0: a page the window has passed; its keys weigh nothing
#pragma unroll
        for (int i = 0; i < KPER; ++i) {
            const int pc = tid + i * 256;
            const int c = pc / (TK * (D / 8)), rest = pc % (TK * (D / 8)), key = rest / (D / 8), piece = rest % (D / 8);
            kreg[i] = zero4;
            if (pc < KPIECES && pg >= 0) kreg[i] = *reinterpret_cast<const uint4*>(kc + (((size_t)pg * NC + c) * page + off + key) * D + piece * 8);
        }
#pragma unroll
        for (int i = 0; i < VPER; ++i) {
            const int pc = tid + i * 256;
            const int c = pc / (D * (TK / 8)), rest = pc % (D * (TK / 8)), row = rest / (TK / 8), piece = rest % (TK / 8);
            vreg[i] = zero4;
            if (pc < VPIECES && pg >= 0) vreg[i] = *reinterpret_cast<const uint4*>(vc + (((size_t)pg * NC + c) * D + row) * page + off + piece * 8);
        }
    };
    // The first `keep_first` keys of the sequence stay seen below the window's edge: their tiles go first (in the chunked form:
    // in chunk 0), then the tiles from the window's edge on.  Tile i of the walk begins at key tile_key(i).
    int n_pre = 0;
    if (keep_first > 0 && (chunk_keys == 0 || blockIdx.z == 0)) {
        const int edge = lo_first & ~(TK - 1);                   // (the window's tiles begin here; kept keys from here on are theirs)
        n_pre = (min(keep_first, edge) + TK - 1) / TK;
    }
    const int n_main = kb_begin <= kb_end ? (kb_end - kb_begin) / TK + 1 : 0;
    auto tile_key = [&](int i) { return i < n_pre ? i * TK : kb_begin + (i - n_pre) * TK; };
    if (n_pre + n_main > 0) fetch(tile_key(0));
    for (int ti = 0; ti < n_pre + n_main; ++ti) {
        const int kb = tile_key(ti);
        __syncthreads();                                         // the tile before this one has been read by every wave
#pragma unroll
        for (int i = 0; i < KPER; ++i) {
            const int pc = tid + i * 256;
            const int c = pc / (TK * (D / 8)), rest = pc % (TK * (D / 8)), key = rest / (D / 8), piece = rest % (D / 8);
            if (pc < KPIECES) *reinterpret_cast<uint4*>(Ks + (c * TK + key) * KROW + piece * 8) = kreg[i];
        }
#pragma unroll
        for (int i = 0; i < VPER; ++i) {
            const int pc = tid + i * 256;
            const int c = pc / (D * (TK / 8)), rest = pc % (D * (TK / 8)), row = rest / (TK / 8), piece = rest % (TK / 8);
            if (pc < VPIECES) *reinterpret_cast<uint4*>(Vs + (c * D + row) * VROW + piece * 8) = vreg[i];
        }
        __syncthreads();
        if (ti + 1 < n_pre + n_main) fetch(tile_key(ti + 1));
        // head by head (a version that read every key and value fragment from LDS once for all heads of a wave kept more
        // registers live and measured slower: 455 against 374 us a prompt step at 32 heads of 128)
#pragma unroll
        for (int i = 0; i < HPW; ++i) {
            if (!head_ok[i]) continue;                           // (uniform over the wave)
            hx_f32x4 S[NS];
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                S[s] = hx_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < NC; ++c)
#pragma unroll
                    for (int ks = 0; ks < D32; ++ks) {
                        const uint4 a = *reinterpret_cast<const uint4*>(Ks + (c * TK + s * 16 + r) * KROW + ks * 32 + g4 * 8);
                        S[s] = hx_mfma(a, qf[i][c][ks], S[s]);
                    }
            }
            // this lane: token r, keys kb + 16 s + 4 g4 + j
            float sc[4 * NS];
            float mx = HX_NEG;
#pragma unroll
            for (int s = 0; s < NS; ++s)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int key = kb + s * 16 + g4 * 4 + j;
                    const bool seen = tok_ok && key <= p_tok && (key >= lo_tok || key < keep_first);
                    sc[s * 4 + j] = seen ? S[s][j] * scale_log2e : HX_NEG;
                    mx = fmaxf(mx, sc[s * 4 + j]);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m_run[i], mx);
            const float corr = __builtin_amdgcn_exp2f(m_run[i] - m_new);
            float pw[4 * NS], sum = 0.f;
#pragma unroll
            for (int j = 0; j < 4 * NS; ++j) {
                pw[j] = sc[j] > 0.5f * HX_NEG ? __builtin_amdgcn_exp2f(sc[j] - m_new) : 0.f;
                sum += pw[j];
            }
            l_run[i] = l_run[i] * corr + sum;                    // (this lane's share; the four lanes of a token are summed at the end)
            m_run[i] = m_new;
            // the float weights enter the second product as two bfloat16 terms (the rounded weight and what the rounding
            // left), so 16 bits of each weight count instead of 8; a product takes 32 keys: subtiles 2 u and 2 u + 1
            uint4 pb[NP], pb_lo[NP];
#pragma unroll
            for (int u = 0; u < NP; ++u) {
                float pl[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) pl[j] = pw[8 * u + j] - to_f32(from_f32<bf16>(pw[8 * u + j]));
                pb[u] = make_uint4(hx_pack(pw[8 * u], pw[8 * u + 1]), hx_pack(pw[8 * u + 2], pw[8 * u + 3]), hx_pack(pw[8 * u + 4], pw[8 * u + 5]),
                                   hx_pack(pw[8 * u + 6], pw[8 * u + 7]));
                pb_lo[u] = make_uint4(hx_pack(pl[0], pl[1]), hx_pack(pl[2], pl[3]), hx_pack(pl[4], pl[5]), hx_pack(pl[6], pl[7]));
            }
            const int c_h = head[i] / per;
#pragma unroll
            for (int b = 0; b < 2 * D32; ++b) {
                const bf16* vrow = Vs + (c_h * D + b * 16 + r) * VROW;
                hx_f32x4 o = O[i][b];
                o[0] *= corr; o[1] *= corr; o[2] *= corr; o[3] *= corr;
#pragma unroll
                for (int u = 0; u < NP; ++u) {
                    const uint2 v0 = *reinterpret_cast<const uint2*>(vrow + 32 * u + g4 * 4);          // keys 32 u + 4 g4 .. + 3
                    const uint2 v1 = *reinterpret_cast<const uint2*>(vrow + 32 * u + 16 + g4 * 4);     // keys 32 u + 16 + 4 g4 .. + 3
                    const uint4 va = make_uint4(v0.x, v0.y, v1.x, v1.y);
                    o = hx_mfma(va, pb_lo[u], hx_mfma(va, pb[u], o));
                }
                O[i][b] = o;
            }
        }
    }
#pragma unroll
    for (int i = 0; i < HPW; ++i) {
        if (!head_ok[i]) continue;
        float l = l_run[i];
        l += __shfl_xor(l, 16, 64);
        l += __shfl_xor(l, 32, 64);
        if (chunk_keys > 0) {
            if (HC ? lane_ok[i] : r == 0) {      // (a single token: column 0, or every column its head)
                float* dst = ws + (((size_t)blockIdx.x * gridDim.z + blockIdx.z) * nh + head[i]) * (D + 4);
#pragma unroll
                for (int b = 0; b < 2 * D32; ++b)
                    *reinterpret_cast<float4*>(dst + b * 16 + g4 * 4) = make_float4(O[i][b][0], O[i][b][1], O[i][b][2], O[i][b][3]);
                if (g4 == 0) { dst[D] = m_run[i]; dst[D + 1] = l; }
            }
            continue;
        }
        if (sink != nullptr) l += __builtin_amdgcn_exp2f(sink[head[i]] * 1.4426950408889634f - m_run[i]);
        const float inv = 1.0f / l;
        if (tok_ok && lane_ok[i] && out_f32) {       // (float rows for a caller that goes on in float: `out` then points to floats)
            float* orow = reinterpret_cast<float*>(out) + (size_t)tok * out_stride + (size_t)head[i] * D;
#pragma unroll
            for (int b = 0; b < 2 * D32; ++b) {
                const hx_f32x4 o = O[i][b];
                *reinterpret_cast<float4*>(orow + b * 16 + g4 * 4) = make_float4(o[0] * inv, o[1] * inv, o[2] * inv, o[3] * inv);
            }
        } else if (tok_ok && lane_ok[i]) {
            bf16* orow = out + (size_t)tok * out_stride + (size_t)head[i] * D;
#pragma unroll
            for (int b = 0; b < 2 * D32; ++b) {
                const hx_f32x4 o = O[i][b];
                *reinterpret_cast<uint2*>(orow + b * 16 + g4 * 4) = make_uint2(hx_pack(o[0] * inv, o[1] * inv), hx_pack(o[2] * inv, o[3] * inv));
            }
        }
    }
}

// the chunks' partial results of a single token and head folded in order, the sink's term, the division
__global__ void __launch_bounds__(128)
attn_headmix_merge_kernel(bf16* __restrict__ out, const float* __restrict__ ws, const int* __restrict__ singles,
                          const float* __restrict__ sink, int nh, int D, int nz, int out_stride, int out_f32) {
    const int item = blockIdx.x, h = blockIdx.y, e = threadIdx.x;
    const int t = singles != nullptr ? singles[item] : item;
    if (t < 0 || e >= D) return;
    float M = HX_NEG, L = 0.f, A = 0.f;
    for (int z = 0; z < nz; ++z) {
        const float* src = ws + (((size_t)item * nz + z) * nh + h) * (D + 4);
        const float m = src[D], l = src[D + 1];
        const float Mn = fmaxf(M, m);
        const float a = __builtin_amdgcn_exp2f(M - Mn), b = __builtin_amdgcn_exp2f(m - Mn);
        L = fmaf(L, a, l * b);
        A = fmaf(A, a, src[e] * b);
        M = Mn;
    }
    if (sink != nullptr) L += __builtin_amdgcn_exp2f(sink[h] * 1.4426950408889634f - M);
    if (out_f32) reinterpret_cast<float*>(out)[(size_t)t * out_stride + (size_t)h * D + e] = A / L;
    else out[(size_t)t * out_stride + (size_t)h * D + e] = from_f32<bf16>(A / L);
}

extern "C" int ilm_attn_headmix_mfma_ok(int nh, int nkv, int d, int page) {
    return nh > 0 && nkv > 0 && nh % nkv == 0 && (nkv == 1 || nkv == 2 || nkv == 4) && d % 32 == 0 && d >= 32 && d <= 128 &&
           page % 32 == 0;
}

// qx [T, nh, nkv, d] from ilm_headmix_queries; tiles [n_tiles, 2] = (first row, count <= 8) and n_singles single rows
// (`singles` null: rows 0 .. n_singles - 1; an entry -1 or a count 0 names nothing); seg_offsets (may be null): the first row
// of every request of the step and the end of the last, with which tiles cut 8 by 8 from a request's first row are served
// two at a time
extern "C" int ilm_attn_headmix_mfma(void* out, const void* qx, const void* kc, const void* vc, const void* block_tables,
                                     const void* seg, const void* pos, const void* tiles, int n_tiles, const void* singles,
                                     int n_singles, const void* sink, int nh, int nkv, int d, int page, int max_blocks,
                                     int out_stride, float scale, int window, void* ws, int nz, int chunk_keys,
                                     const void* seg_offsets, int keep_first, int out_f32, hipStream_t stream) {
    ILM_REQUIRE(keep_first >= 0, "attn_headmix_mfma: %d kept first tokens", keep_first);
    // single tokens whose heads come in groups of a multiple of 16: heads as the products' columns
    // (a block of 16 columns must lie in one key/value group: one group in all, or groups of a multiple of 16 heads)
    const bool hc = n_tiles == 0 && (nkv == 1 || (nh % 16 == 0 && (nh / (nkv > 0 ? nkv : 1)) % 16 == 0));
    // ws != null (single tokens only): nz chunks of chunk_keys keys a token, float [n_singles][nz][nh][d + 4]
    ILM_REQUIRE(ws == nullptr || (n_tiles == 0 && nz >= 1 && nz <= 65535 && chunk_keys > 0 && chunk_keys % 64 == 0),
                "attn_headmix_mfma: chunks are for single tokens, in multiples of 64 keys");
    if (ws == nullptr) { nz = 1; chunk_keys = 0; }
    ILM_REQUIRE(n_tiles >= 0 && n_singles >= 0 && n_tiles + n_singles > 0 && max_blocks > 0, "attn_headmix_mfma: bad sizes");
    ILM_REQUIRE(ilm_attn_headmix_mfma_ok(nh, nkv, d, page), "attn_headmix_mfma: %d heads in %d groups of %d, pages of %d", nh, nkv, d, page);
    ILM_REQUIRE(!out_f32 || ((uintptr_t)out & 15) == 0, "attention_headmix_mfma: float rows must be 16-byte aligned");
    ILM_REQUIRE(out_stride % 4 == 0 && ((uintptr_t)out & 7) == 0 && ((uintptr_t)qx & 15) == 0 && ((uintptr_t)kc & 15) == 0 &&
                ((uintptr_t)vc & 15) == 0, "attn_headmix_mfma: rows must be 16-byte / 8-byte aligned");
    const float scale_log2e = scale * 1.4426950408889634f;
#define HX_LAUNCH(D32_, NC_, HPW_)                                                                                         \
    if (hc) HX_LAUNCH_TK(D32_, NC_, 1, 32, true) else HX_LAUNCH_TK(D32_, NC_, HPW_, 32, false)
#define HX_LAUNCH_TK(D32_, NC_, HPW_, TK_, HC_)                                                                            \
    {                                                                                                                      \
        auto kern = attn_headmix_mfma_kernel<D32_, NC_, HPW_, TK_, HC_>;                                                   \
        const int shm = NC_ * TK_ * (D32_ * 32 + 8) * 2 + NC_ * D32_ * 32 * (TK_ + 8) * 2;                                 \
        if (shm > 48 * 1024) {                                                                                             \
            hipError_t e_ = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, shm);       \
            ILM_REQUIRE(e_ == hipSuccess, "attn_headmix_mfma: %d bytes of LDS refused: %s", shm, hipGetErrorString(e_));   \
        }                                                                                                                  \
        dim3 grid(n_tiles + n_singles, HC_ ? (nh + 63) / 64 : (nh + 4 * HPW_ - 1) / (4 * HPW_), nz);                       \
        kern<<<grid, 256, shm, stream>>>((bf16*)out, (const bf16*)qx, (const bf16*)kc, (const bf16*)vc,                    \
                                         (const int*)block_tables, (const int*)seg, (const int*)pos, (const int*)tiles,    \
                                         n_tiles, (const int*)singles, (const float*)sink, nh, page, max_blocks,           \
                                         out_stride, scale_log2e, window, (float*)ws, chunk_keys,                          \
                                         (const int*)seg_offsets, keep_first, out_f32);                                    \
    }
#define HX_BY_NC(D32_)                                                      \
    switch (nkv) {                                                          \
        case 1: if (D32_ <= 2) HX_LAUNCH(D32_, 1, 4) else HX_LAUNCH(D32_, 1, 1) break; \
        case 2: if (D32_ <= 2) HX_LAUNCH(D32_, 2, 4) else HX_LAUNCH(D32_, 2, 1) break; \
        default: if (D32_ <= 2) HX_LAUNCH(D32_, 4, 2) else HX_LAUNCH(D32_, 4, 1) break; \
    }
    switch (d / 32) {
        case 1: HX_BY_NC(1) break;
        case 2: HX_BY_NC(2) break;
        case 3: HX_BY_NC(3) break;
        default: HX_BY_NC(4) break;
    }
#undef HX_BY_NC
#undef HX_LAUNCH
#undef HX_LAUNCH_TK
    ILM_LAUNCH_CHECK("attn_headmix_mfma");
    if (ws != nullptr) {
        attn_headmix_merge_kernel<<<dim3(n_singles, nh), 128, 0, stream>>>((bf16*)out, (const float*)ws, (const int*)singles,
                                                                           (const float*)sink, nh, d, nz, out_stride, out_f32);
        ILM_LAUNCH_CHECK("attn_headmix_mfma (merge)");
    }
    return 0;
}
