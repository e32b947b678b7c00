// Attention through latents: what lies between the down projections and the attention kernel.
//
// A layer of this kind projects a row down twice: to a query latent of `q_rank` numbers, and to a key/value latent of `kv_rank`
// numbers with `rot` more that are one rotated key part for all heads.  Both latents are RMS-normed with weights of their own.
// Only the normed key/value latent c and the rotated part are cached, nothing per head, because with the up projections folded
// into the query (q' = W_uk^T q per head) and into the output (o = W_uv sum_j p_j c_j) the latent is key and value at once:
//     score_j = q' . c_j + q_rot . k_rot_j          out = sum_j softmax(score)_j c_j
// A page holds its places' keys [place][kv_rank + rot] and, behind them, the latent once more with the places innermost
// [kv_rank][place]: the layout of a layer with one key/value head whose values are shorter than its keys, which every attention
// kernel reads, and both operands of the matrix instructions come out of memory as they lie.
// The rotation here turns neighbouring channels, the pair (2i, 2i + 1) by pos * f_i.
//
//   latent_prepare   one wave per (row, which): the query latent normed into the rows the up projection reads; the key/value
//                    latent normed and the rotated part turned, both written to the row's place in its page
//   latent_queries   one wave per (row, head): a head's unrotated channels into the rows the folding product reads, its
//                    rotated channels turned and written behind the place where that product puts q'
//   heads_product    out[t, h, :] = a[t, h, :] W_h^T for every head in one launch (the folding of W_uk into the queries and the
//                    product with W_uv behind the attention), on the matrix cores
//   latent_attention one wave per (row, 16 heads, share of the context): all heads read the same keys, so 16 of them are the
//                    columns of one matrix instruction even for a single decoded row; for the rows of prompts a workgroup takes a
//                    few consecutive rows with all their heads and stages the keys they see once in LDS
#include "common.h"

namespace {

template <typename TW, typename TA, typename TC>
__global__ __launch_bounds__(64) void latent_prepare_kernel(const float* __restrict__ proj, long ld, int q_rank, int kv_rank, int rot,
                                                           const TW* __restrict__ q_norm, const TW* __restrict__ kv_norm, float eps,
                                                           const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                           const int* __restrict__ pos, const int* __restrict__ slot, const int* __restrict__ table,
                                                           int table_stride, TA* __restrict__ cq, long ldcq, TC* __restrict__ cache, long page_stride,
                                                           int page_size) {
    const int t = blockIdx.x, lane = threadIdx.x;
    const bool query = blockIdx.y == 0;
    const float* src = proj + (size_t)t * ld + (query ? 0 : q_rank);
    const int n = query ? q_rank : kv_rank;
    const TW* w = query ? q_norm : kv_norm;
    float ss = 0.f;
    for (int d = lane; d < n; d += 64) ss = fmaf(src[d], src[d], ss);
    const float r = 1.0f / sqrtf(wave_sum(ss) / (float)n + eps);
    if (query) {
        for (int d = lane; d < n; d += 64) store_f32(cq, (size_t)t * ldcq + d, load_f32(w, d) * (r * src[d]));
        return;
    }
    const int p = pos[t];
    const long page = table[(size_t)slot[t] * table_stride + p / page_size];
    TC* dst = cache + page * page_stride + (size_t)(p % page_size) * (kv_rank + rot);
    TC* as_value = cache + page * page_stride + (size_t)page_size * (kv_rank + rot) + p % page_size;      // [kv_rank][place]
    for (int d = lane; d < n; d += 64) {
        const float c = load_f32(w, d) * (r * src[d]);
        store_f32(dst, d, c);
        store_f32(as_value, (size_t)d * page_size, c);
    }
    for (int i = lane; i < rot / 2; i += 64) {
        const float u = src[kv_rank + 2 * i], v = src[kv_rank + 2 * i + 1];
        const float c = cos_t[(size_t)t * (rot / 2) + i], s = sin_t[(size_t)t * (rot / 2) + i];
        store_f32(dst, kv_rank + 2 * i, u * c - v * s);
        store_f32(dst, kv_rank + 2 * i + 1, v * c + u * s);
    }
}

template <typename TA, typename TC>
__global__ __launch_bounds__(64) void latent_queries_kernel(const float* __restrict__ q, long ldq, const float* __restrict__ cos_t,
                                                           const float* __restrict__ sin_t, TA* __restrict__ plain, long ld_plain,
                                                           TC* __restrict__ folded, long ld_folded, int n_heads, int dim, int rot, int kv_rank) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float* src = q + (size_t)t * ldq + (size_t)h * (dim + rot);
    for (int d = lane; d < dim; d += 64) store_f32(plain, (size_t)t * ld_plain + (size_t)h * dim + d, src[d]);
    TC* dst = folded + (size_t)t * ld_folded + (size_t)h * (kv_rank + rot) + kv_rank;
    for (int i = lane; i < rot / 2; i += 64) {
        const float u = src[dim + 2 * i], v = src[dim + 2 * i + 1];
        const float c = cos_t[(size_t)t * (rot / 2) + i], s = sin_t[(size_t)t * (rot / 2) + i];
        store_f32(dst, 2 * i, u * c - v * s);
        store_f32(dst, 2 * i + 1, v * c + u * s);
    }
}

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ bf16x8 as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8, v); }
__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

// out[t, h*n_out + n] = sum_k a[t, h*k_dim + k] * w[h][n][k], bfloat16 operands, 32-bit sums.  One wave per (16 rows, head, 64
// columns): the operands of the 16x16x32 matrix instruction are 16-byte pieces of a's and w's rows as they lie in memory.
template <typename TO>
__global__ __launch_bounds__(64) void heads_product_kernel(const bf16_t* __restrict__ a, long lda, const bf16_t* __restrict__ w, TO* __restrict__ out, long ldo,
                                                          long out_head_stride, int n_rows, int k_dim, int n_out) {
    const int lane = threadIdx.x, r = lane & 15, q4 = lane >> 4;
    const int row0 = blockIdx.x * 16, h = blockIdx.y, col0 = blockIdx.z * 64;
    const int row = min(row0 + r, n_rows - 1);
    const bf16_t* arow = a + (size_t)row * lda + (size_t)h * k_dim;
    const bf16_t* wh = w + (size_t)h * n_out * k_dim;
    floatx4 acc[4] = {floatx4{}, floatx4{}, floatx4{}, floatx4{}};
    for (int k0 = 0; k0 < k_dim; k0 += 32) {
        const int k = k0 + 8 * q4;
        const bool in = k < k_dim;                       // (k_dim is a multiple of 8: a piece is inside or outside as a whole)
        uint4 av = *reinterpret_cast<const uint4*>(arow + (in ? k : 0));
        if (!in) av = uint4{0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = min(col0 + 16 * j + r, n_out - 1);
            uint4 wv = *reinterpret_cast<const uint4*>(wh + (size_t)col * k_dim + (in ? k : 0));
            if (!in) wv = uint4{0, 0, 0, 0};
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(av), as_bf16x8(wv), acc[j], 0, 0, 0);
        }
    }
    // element v of acc[j]: row row0 + 4*q4 + v, column col0 + 16*j + r
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int col = col0 + 16 * j + r;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int t = row0 + 4 * q4 + v;
            if (t < n_rows && col < n_out) store_f32(out, (size_t)t * ldo + (size_t)h * out_head_stride + col, acc[j][v]);
        }
    }
}

// Attention over the latent pages on the matrix cores.  One wave: row t, heads 16 hg .. 16 hg + 15, share `sp` of the row's
// context.  Tiles of 32 positions (two blocks of 16, each inside one page): S^T = K Q^T puts a position's scores for the 16 heads
// into one lane group, so that a head's maximum and sum are a lane's own plus two exchanges; the probabilities, as they lie, are
// the second operand of O^T = V^T P^T.  KS = key channels / 32 (rounded up: pieces beyond the key are zeros), DT = value channels / 16.
// Shares of one row meet in `part` ([row][head][share]{m, l, o[vd]}, 32-bit) and `latent_merge_kernel` adds them; with one share
// the wave writes the heads' outputs itself.  `rows`: the step's rows that this launch serves (nullptr: all, in order).
template <int KS, int DT>
__global__ __launch_bounds__(64) void latent_attention_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ cache, bf16_t* __restrict__ out,
                                                             float* __restrict__ part, const int* __restrict__ rows, const int* __restrict__ pos,
                                                             const int* __restrict__ slot, const int* __restrict__ table, int table_stride, long page_stride,
                                                             int page_size, int n_heads, int kd, int vd, int window, float scale2, int n_splits) {
    const int lane = threadIdx.x, r = lane & 15, q4 = lane >> 4;
    const int t = rows ? rows[blockIdx.x] : blockIdx.x, hg = blockIdx.y, sp = blockIdx.z;
    const int head = hg * 16 + r;
    const bool head_ok = head < n_heads;
    const int p = pos[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int* tab = table + (size_t)slot[t] * table_stride;
    // this share's tiles
    const int first_tile = lo >> 5, n_tiles = (p >> 5) - first_tile + 1;
    const int per = (n_tiles + n_splits - 1) / n_splits;
    const int tile0 = first_tile + sp * per, tile1 = min(tile0 + per, first_tile + n_tiles);
    const long v_plane = (long)page_size * kd;

    bf16x8 qreg[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int c = 32 * ks + 8 * q4;
        uint4 v = *reinterpret_cast<const uint4*>(q + ((size_t)t * n_heads + (head_ok ? head : 0)) * kd + (c < kd ? c : 0));
        if (!head_ok || c >= kd) v = uint4{0, 0, 0, 0};
        qreg[ks] = as_bf16x8(v);
    }
    floatx4 o[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i) o[i] = floatx4{};
    float m = -INFINITY, l = 0.f;

    for (int tile = tile0; tile < tile1; ++tile) {
        const int kv0 = tile << 5;
        const bf16_t* page[2];
        int place[2];
#pragma unroll
        for (int b = 0; b < 2; ++b) {                    // a block that lies outside what the row sees is read from a place that it does see
            const int j0 = min(max(kv0 + 16 * b, lo & ~15), p & ~15);
            page[b] = cache + (long)tab[j0 / page_size] * page_stride;
            place[b] = j0 % page_size;
        }
        floatx4 s[2];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            s[b] = floatx4{};
            const bf16_t* krow = page[b] + (size_t)(place[b] + r) * kd;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const int c = 32 * ks + 8 * q4;
                uint4 kv = *reinterpret_cast<const uint4*>(krow + (c < kd ? c : 0));
                if (c >= kd) kv = uint4{0, 0, 0, 0};
                s[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kv), qreg[ks], s[b], 0, 0, 0);
            }
        }
        // element v of s[b]: position kv0 + 16*b + 4*q4 + v, head r
        float mx = -INFINITY;
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int j = kv0 + 16 * b + 4 * q4 + v;
                s[b][v] = (j >= lo && j <= p) ? s[b][v] * scale2 : -INFINITY;
                mx = fmaxf(mx, s[b][v]);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m, mx);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float corr = exp2_fast(m - m_use);
        float sum = 0.f;
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                s[b][v] = exp2_fast(s[b][v] - m_use);
                sum += s[b][v];
            }
        sum += __shfl_xor(sum, 16, 64);
        sum += __shfl_xor(sum, 32, 64);
        l = l * corr + sum;
        m = m_new;
        const uint4 pb = {f32x2_to_bf16x2(s[0][0], s[0][1]), f32x2_to_bf16x2(s[0][2], s[0][3]), f32x2_to_bf16x2(s[1][0], s[1][1]), f32x2_to_bf16x2(s[1][2], s[1][3])};
        // a block whose positions are all masked was read from another block's place: its probabilities are zeros, which is all that matters
#pragma unroll
        for (int i = 0; i < DT; ++i) {
            const int c = 16 * i + r;
            const size_t ch = (size_t)(c < vd ? c : 0) * page_size;
            uint2 v0 = *reinterpret_cast<const uint2*>(page[0] + v_plane + ch + place[0] + 4 * q4);
            uint2 v1 = *reinterpret_cast<const uint2*>(page[1] + v_plane + ch + place[1] + 4 * q4);
            if (c >= vd) v0 = v1 = uint2{0, 0};
#pragma unroll
            for (int v = 0; v < 4; ++v) o[i][v] *= corr;
            o[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(uint4{v0.x, v0.y, v1.x, v1.y}), as_bf16x8(pb), o[i], 0, 0, 0);
        }
    }
    // element v of o[i]: channel 16*i + 4*q4 + v, head r
    if (!head_ok) return;
    if (n_splits == 1) {
        const float inv = 1.0f / l;                      // (a row always sees itself: l > 0)
#pragma unroll
        for (int i = 0; i < DT; ++i)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int c = 16 * i + 4 * q4 + v;
                if (c < vd) out[((size_t)t * n_heads + head) * vd + c] = f32_to_bf16(o[i][v] * inv);
            }
        return;
    }
    float* mine = part + (((size_t)blockIdx.x * n_heads + head) * n_splits + sp) * (vd + 2);
    if (q4 == 0) { mine[0] = m; mine[1] = l; }
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int c = 16 * i + 4 * q4 + v;
            if (c < vd) mine[2 + c] = o[i][v];
        }
}

// The shares of one (row, head): out = sum_s 2^(m_s - m) o_s / sum_s 2^(m_s - m) l_s.  Lane s fetches share s's maximum and sum (all
// at once, not one behind the other); the weights wait in LDS; a lane then adds its channels over the shares, in their order, eight
// loads in flight.
__global__ __launch_bounds__(64) void latent_merge_kernel(const float* __restrict__ part, bf16_t* __restrict__ out, const int* __restrict__ rows, int n_heads,
                                                         int vd, int n_splits) {
    __shared__ float weight[64];
    const size_t rh = blockIdx.x;
    const size_t to = (size_t)(rows ? rows[blockIdx.x / n_heads] : blockIdx.x / n_heads) * n_heads + blockIdx.x % n_heads;
    const int lane = threadIdx.x;
    const float* mine = part + rh * n_splits * (vd + 2);
    const float ms = lane < n_splits ? mine[(size_t)lane * (vd + 2)] : -INFINITY;
    const float ls = lane < n_splits ? mine[(size_t)lane * (vd + 2) + 1] : 0.f;
    const float m = wave_max(ms);
    const float w = ms == -INFINITY ? 0.f : exp2_fast(ms - m);
    const float inv = 1.0f / wave_sum(w * ls);
    weight[lane] = w;
    __syncthreads();
    for (int c = lane; c < vd; c += 64) {
        float acc = 0.f;
        int s = 0;
        for (; s + 8 <= n_splits; s += 8) {
            float v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = mine[(size_t)(s + e) * (vd + 2) + 2 + c];
#pragma unroll
            for (int e = 0; e < 8; ++e) acc = fmaf(weight[s + e], v[e], acc);
        }
        for (; s < n_splits; ++s) acc = fmaf(weight[s], mine[(size_t)s * (vd + 2) + 2 + c], acc);
        out[to * vd + c] = f32_to_bf16(acc * inv);
    }
}

// The rows of prompts: a workgroup takes TR consecutive rows of one request (a piece of one of the attention plan's tiles) and all
// their heads, a wave per (row, 16 heads) as above, and the tiles of 32 positions that any of its rows sees are staged once in LDS
// for all of them: the keys [32][key channels, padded so that 16 rows' 16-byte reads fall into different banks], the values
// [value channels][32 places + 8].  Every wave masks by its own row's position and window and skips the tiles it sees nothing of;
// what a workgroup fetches from the L2 is shared by TR rows x all heads instead of 16 heads.
template <int KS, int DT, bool AHEAD>
__global__ __launch_bounds__(512) void latent_attention_tiles_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ cache, bf16_t* __restrict__ out,
                                                                    const int4* __restrict__ tiles, int pieces_per_tile, int TR, int HG,
                                                                    const int* __restrict__ table, int table_stride, long page_stride, int page_size,
                                                                    int n_heads, int kd, int vd, int window, float scale2) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    constexpr int KP = KS * 32 + 8, VP = 40;
    bf16_t* Ks = reinterpret_cast<bf16_t*>(lds);         // [32][KP]
    bf16_t* Vs = Ks + 32 * KP;                           // [DT * 16][VP]
    const int tid = threadIdx.x, NT = blockDim.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, q4 = lane >> 4;
    const int4 tile = tiles[blockIdx.x / pieces_per_tile];
    const int piece = blockIdx.x % pieces_per_tile;
    const int row0 = tile.x + piece * TR, n_tok = min(TR, tile.x + tile.y - row0);
    if (n_tok <= 0) return;                              // (the whole workgroup, before any barrier)
    const int p_first = tile.z + piece * TR, p_last = p_first + n_tok - 1;
    const int lo_all = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
    const int* tab = table + (size_t)tile.w * table_stride;
    const long v_plane = (long)page_size * kd;
    for (int i = tid; i < (32 * KP + DT * 16 * VP) / 2; i += NT) reinterpret_cast<uint32_t*>(lds)[i] = 0;      // channels beyond the key's and the value's stay zeros

    const int ti = min(wave / HG, n_tok - 1), hg = wave % HG;
    const bool tok_ok = wave / HG < n_tok;
    const int t = row0 + ti, p = p_first + ti;
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int head = hg * 16 + r;
    const bool head_ok = tok_ok && head < n_heads;
    bf16x8 qreg[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int c = 32 * ks + 8 * q4;
        uint4 v = *reinterpret_cast<const uint4*>(q + ((size_t)t * n_heads + (head < n_heads ? head : 0)) * kd + (c < kd ? c : 0));
        if (!head_ok || c >= kd) v = uint4{0, 0, 0, 0};
        qreg[ks] = as_bf16x8(v);
    }
    floatx4 o[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i) o[i] = floatx4{};
    float m = -INFINITY, l = 0.f;
    const int k_pieces = kd >> 3;
    // A tile on its way: every position's key in 16-byte pieces, every value channel's 32 places in four.  With AHEAD the next
    // tile is asked for into registers before this one is worked on (workgroups have 320 threads or more: a thread brings at most
    // KPER + VPER pieces); without (the largest sizes, whose registers are spoken for) a tile is fetched when its turn comes.
    constexpr int KPER = (32 * KS * 4 + 319) / 320, VPER = (DT * 16 * 4 + 319) / 320;
    uintx4 k_reg[AHEAD ? KPER : 1], v_reg[AHEAD ? VPER : 1];
    auto k_source = [&](int kv0, int idx) {
        const int key = idx / k_pieces, piece8 = idx % k_pieces;
        const int j = min(max(kv0 + key, lo_all), p_last);               // (a position nobody sees is read from one that somebody does)
        return cache + (long)tab[j / page_size] * page_stride + (size_t)(j % page_size) * kd + 8 * piece8;
    };
    auto v_source = [&](int kv0, int idx) {
        const int c = idx >> 2, b = (idx >> 1) & 1, e = idx & 1;
        const int j0 = min(max(kv0 + 16 * b, lo_all & ~15), p_last & ~15);
        return cache + (long)tab[j0 / page_size] * page_stride + v_plane + (size_t)c * page_size + j0 % page_size + 8 * e;
    };
    const int tk_last = p_last >> 5;
    {
        if constexpr (AHEAD) {
#pragma unroll
            for (int e = 0; e < KPER; ++e) k_reg[e] = *reinterpret_cast<const uintx4*>(k_source((lo_all >> 5) << 5, min(tid + e * NT, 32 * k_pieces - 1)));
#pragma unroll
            for (int e = 0; e < VPER; ++e) v_reg[e] = *reinterpret_cast<const uintx4*>(v_source((lo_all >> 5) << 5, min(tid + e * NT, vd * 4 - 1)));
        }
    }
    __syncthreads();

    for (int tk = lo_all >> 5; tk <= tk_last; ++tk) {
        const int kv0 = tk << 5;
        if constexpr (AHEAD) {
#pragma unroll
            for (int e = 0; e < KPER; ++e) {
                const int idx = tid + e * NT;
                if (idx < 32 * k_pieces) *reinterpret_cast<uintx4*>(Ks + (idx / k_pieces) * KP + 8 * (idx % k_pieces)) = k_reg[e];
            }
#pragma unroll
            for (int e = 0; e < VPER; ++e) {
                const int idx = tid + e * NT;
                if (idx < vd * 4) *reinterpret_cast<uintx4*>(Vs + (idx >> 2) * VP + 16 * ((idx >> 1) & 1) + 8 * (idx & 1)) = v_reg[e];
            }
        } else {
            for (int idx = tid; idx < 32 * k_pieces; idx += NT)
                *reinterpret_cast<uint4*>(Ks + (idx / k_pieces) * KP + 8 * (idx % k_pieces)) = *reinterpret_cast<const uint4*>(k_source(kv0, idx));
            for (int idx = tid; idx < vd * 4; idx += NT)
                *reinterpret_cast<uint4*>(Vs + (idx >> 2) * VP + 16 * ((idx >> 1) & 1) + 8 * (idx & 1)) = *reinterpret_cast<const uint4*>(v_source(kv0, idx));
        }
        __syncthreads();
        if (tk < tk_last) {
        if constexpr (AHEAD) {
#pragma unroll
            for (int e = 0; e < KPER; ++e) k_reg[e] = *reinterpret_cast<const uintx4*>(k_source(kv0 + 32, min(tid + e * NT, 32 * k_pieces - 1)));
#pragma unroll
            for (int e = 0; e < VPER; ++e) v_reg[e] = *reinterpret_cast<const uintx4*>(v_source(kv0 + 32, min(tid + e * NT, vd * 4 - 1)));
        }
        }
        if (tok_ok && tk >= (lo >> 5) && tk <= (p >> 5)) {
            floatx4 s[2];
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                s[b] = floatx4{};
                const bf16_t* krow = Ks + (16 * b + r) * KP + 8 * q4;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    s[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(*reinterpret_cast<const uint4*>(krow + 32 * ks)), qreg[ks], s[b], 0, 0, 0);
            }
            float mx = -INFINITY;
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int j = kv0 + 16 * b + 4 * q4 + v;
                    s[b][v] = (j >= lo && j <= p) ? s[b][v] * scale2 : -INFINITY;
                    mx = fmaxf(mx, s[b][v]);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m, mx);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            const float corr = exp2_fast(m - m_use);
            float sum = 0.f;
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    s[b][v] = exp2_fast(s[b][v] - m_use);
                    sum += s[b][v];
                }
            sum += __shfl_xor(sum, 16, 64);
            sum += __shfl_xor(sum, 32, 64);
            l = l * corr + sum;
            m = m_new;
            const uint4 pb = {f32x2_to_bf16x2(s[0][0], s[0][1]), f32x2_to_bf16x2(s[0][2], s[0][3]), f32x2_to_bf16x2(s[1][0], s[1][1]), f32x2_to_bf16x2(s[1][2], s[1][3])};
#pragma unroll
            for (int i = 0; i < DT; ++i) {
                const bf16_t* vrow = Vs + (16 * i + r) * VP + 4 * q4;
                const uint2 v0 = *reinterpret_cast<const uint2*>(vrow), v1 = *reinterpret_cast<const uint2*>(vrow + 16);
#pragma unroll
                for (int v = 0; v < 4; ++v) o[i][v] *= corr;
                o[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(uint4{v0.x, v0.y, v1.x, v1.y}), as_bf16x8(pb), o[i], 0, 0, 0);
            }
        }
        __syncthreads();
    }
    if (!head_ok) return;
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int c = 16 * i + 4 * q4 + v;
            if (c < vd) out[((size_t)t * n_heads + head) * vd + c] = f32_to_bf16(o[i][v] * inv);
        }
}


}  // namespace

// proj: float32 [n_rows, ld] = [query latent (q_rank) | key/value latent (kv_rank) | rotated key part (rot)]; cos, sin: float32
// [n_rows, rot/2]; cq: [n_rows, ldcq] gets the normed query latent; the cache's pages hold [place][kv_rank + rot], then [kv_rank][place].
GI_API int gi_latent_prepare(const float* proj, long ld, int q_rank, int kv_rank, int rot, const void* q_norm, const void* kv_norm, int norm_dtype,
                             float eps, const float* cos_t, const float* sin_t, const int* pos, const int* slot, const int* table, int table_stride,
                             void* cq, int cq_dtype, long ldcq, void* cache, int cache_dtype, long page_stride, int page_size, int n_rows,
                             hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && q_rank > 0 && kv_rank > 0 && rot >= 0 && rot % 2 == 0, "latent_prepare: bad sizes (rows %d, latents %d and %d, %d rotated channels)",
               n_rows, q_rank, kv_rank, rot);
    GI_REQUIRE(ld >= (long)q_rank + kv_rank + rot && ldcq >= q_rank && page_size > 0 && page_stride >= (long)page_size * (2L * kv_rank + rot),
               "latent_prepare: rows or pages too small for these latents");
    GI_REQUIRE(rot == 0 || (cos_t != nullptr && sin_t != nullptr), "latent_prepare: a rotation needs its cosines and sines");
    dim3 grid(n_rows, 2);
#define GO(TW, TA, TC)                                                                                                                        \
    latent_prepare_kernel<TW, TA, TC><<<grid, 64, 0, stream>>>(proj, ld, q_rank, kv_rank, rot, (const TW*)q_norm, (const TW*)kv_norm, eps, cos_t, sin_t, pos, \
                                                               slot, table, table_stride, (TA*)cq, ldcq, (TC*)cache, page_stride, page_size)
    if (norm_dtype == GI_F32 && cq_dtype == GI_F32 && cache_dtype == GI_F32) GO(float, float, float);
    else if (norm_dtype == GI_BF16 && cq_dtype == GI_BF16 && cache_dtype == GI_BF16) GO(bf16_t, bf16_t, bf16_t);
    else if (norm_dtype == GI_F32 && cq_dtype == GI_BF16 && cache_dtype == GI_BF16) GO(float, bf16_t, bf16_t);
    else if (norm_dtype == GI_F32 && cq_dtype == GI_F32 && cache_dtype == GI_BF16) GO(float, float, bf16_t);
    else if (norm_dtype == GI_BF16 && cq_dtype == GI_F32 && cache_dtype == GI_BF16) GO(bf16_t, float, bf16_t);
    else return gi_fail("latent_prepare: dtypes (%d, %d, %d) are not served", norm_dtype, cq_dtype, cache_dtype);
#undef GO
    GI_CHECK_LAUNCH("latent_prepare");
    return 0;
}

// q: float32 [n_rows, ldq], per head [dim unrotated | rot rotated]; plain: [n_rows, ld_plain] gets the heads' unrotated channels
// [n_heads][dim]; folded: [n_rows, ld_folded], per head [kv_rank + rot], gets the turned channels behind each head's first kv_rank.
GI_API int gi_latent_queries(const float* q, long ldq, const float* cos_t, const float* sin_t, void* plain, int plain_dtype, long ld_plain, void* folded,
                             int folded_dtype, long ld_folded, int n_rows, int n_heads, int dim, int rot, int kv_rank, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_heads > 0 && n_heads <= 65535 && dim > 0 && rot >= 0 && rot % 2 == 0 && kv_rank > 0, "latent_queries: bad sizes (rows %d, heads %d, %d + %d channels)",
               n_rows, n_heads, dim, rot);
    GI_REQUIRE(ldq >= (long)n_heads * (dim + rot) && ld_plain >= (long)n_heads * dim && ld_folded >= (long)n_heads * (kv_rank + rot), "latent_queries: rows too short");
    GI_REQUIRE(rot == 0 || (cos_t != nullptr && sin_t != nullptr), "latent_queries: a rotation needs its cosines and sines");
    dim3 grid(n_rows, n_heads);
#define GO(TA, TC) latent_queries_kernel<TA, TC><<<grid, 64, 0, stream>>>(q, ldq, cos_t, sin_t, (TA*)plain, ld_plain, (TC*)folded, ld_folded, n_heads, dim, rot, kv_rank)
    if (plain_dtype == GI_F32 && folded_dtype == GI_F32) GO(float, float);
    else if (plain_dtype == GI_BF16 && folded_dtype == GI_BF16) GO(bf16_t, bf16_t);
    else if (plain_dtype == GI_F32 && folded_dtype == GI_BF16) GO(float, bf16_t);
    else return gi_fail("latent_queries: dtypes (%d, %d) are not served", plain_dtype, folded_dtype);
#undef GO
    GI_CHECK_LAUNCH("latent_queries");
    return 0;
}

// a: bfloat16 [n_rows, lda], head h's operand in columns [h*k_dim, (h+1)*k_dim); w: bfloat16 [n_heads][n_out][k_dim]; out: [n_rows, ldo],
// head h's result in columns [h*out_head_stride, h*out_head_stride + n_out).
GI_API int gi_heads_product_supports(int k_dim, int n_out) { return k_dim > 0 && n_out > 0 && k_dim % 8 == 0; }

GI_API int gi_heads_product(const void* a, long lda, const void* w, void* out, int out_dtype, long ldo, long out_head_stride, int n_rows, int n_heads, int k_dim,
                            int n_out, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_heads > 0 && n_heads <= 65535 && gi_heads_product_supports(k_dim, n_out), "heads_product: bad sizes (rows %d, heads %d, k %d, n %d; k a multiple of 8)",
               n_rows, n_heads, k_dim, n_out);
    GI_REQUIRE(lda % 8 == 0 && lda >= (long)n_heads * k_dim && ((uintptr_t)a & 15) == 0 && ((uintptr_t)w & 15) == 0 && out_head_stride >= n_out &&
               ldo >= (long)(n_heads - 1) * out_head_stride + n_out, "heads_product: operands must be 16-byte aligned with row strides that are multiples of 8, and rows long enough");
    GI_REQUIRE((n_out + 63) / 64 <= 65535, "heads_product: too many columns");
    dim3 grid((n_rows + 15) / 16, n_heads, (n_out + 63) / 64);
    if (out_dtype == GI_F32) heads_product_kernel<float><<<grid, 64, 0, stream>>>((const bf16_t*)a, lda, (const bf16_t*)w, (float*)out, ldo, out_head_stride, n_rows, k_dim, n_out);
    else if (out_dtype == GI_BF16) heads_product_kernel<bf16_t><<<grid, 64, 0, stream>>>((const bf16_t*)a, lda, (const bf16_t*)w, (bf16_t*)out, ldo, out_head_stride, n_rows, k_dim, n_out);
    else return gi_fail("heads_product: unknown output dtype %d", out_dtype);
    GI_CHECK_LAUNCH("heads_product");
    return 0;
}

// Sizes the matrix-core latent attention takes: keys of up to 576 channels in 16-byte pieces, values of up to 512 channels, pages of whole blocks of 16 places.
GI_API int gi_latent_attention_supports(int kd, int vd, int page_size) {
    return kd > 0 && kd % 8 == 0 && kd <= 576 && vd > 0 && vd <= 512 && vd <= kd && page_size > 0 && page_size % 16 == 0;
}
GI_API long gi_latent_attention_scratch_floats(int n_rows, int n_heads, int vd, int n_splits) {
    return n_splits > 1 ? (long)n_rows * n_heads * n_splits * (vd + 2) : 0;
}

// q: bfloat16 [n_rows, n_heads*kd] (folded queries); cache: bfloat16 pages [place][kd] then [vd][place]; out: bfloat16 [n_rows, n_heads*vd].
// rows: the n_rows rows of the step to serve (nullptr: rows 0 .. n_rows - 1).
GI_API int gi_latent_attention_bf16(const void* q, const void* cache, void* out, float* part, long part_floats, const int* rows, const int* pos, const int* slot,
                                    const int* table, int table_stride, long page_stride, int page_size, int n_rows, int n_heads, int kd, int vd, int window,
                                    float scale, int n_splits, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_heads > 0 && gi_latent_attention_supports(kd, vd, page_size), "latent_attention: sizes (rows %d, heads %d, keys %d, values %d, pages of %d) are not taken",
               n_rows, n_heads, kd, vd, page_size);
    GI_REQUIRE(window >= 0 && n_splits >= 1 && n_splits <= 64 && page_stride >= (long)page_size * (kd + vd) && page_stride % 8 == 0 && ((uintptr_t)cache & 15) == 0 &&
               ((uintptr_t)q & 15) == 0, "latent_attention: bad window, shares, page stride or alignment");
    GI_REQUIRE(part_floats >= gi_latent_attention_scratch_floats(n_rows, n_heads, vd, n_splits) && (n_splits == 1 || part != nullptr), "latent_attention: scratch of %ld floats needed, %ld given",
               gi_latent_attention_scratch_floats(n_rows, n_heads, vd, n_splits), part_floats);
    GI_REQUIRE((long)n_rows * n_heads < 2147483647L && (n_heads + 15) / 16 <= 65535, "latent_attention: too many rows or heads");
    dim3 grid(n_rows, (n_heads + 15) / 16, n_splits);
    const float scale2 = scale * 1.4426950408889634f;
#define GO(KS, DT)                                                                                                                                      \
    latent_attention_kernel<KS, DT><<<grid, 64, 0, stream>>>((const bf16_t*)q, (const bf16_t*)cache, (bf16_t*)out, part, rows, pos, slot, table, table_stride, \
                                                             page_stride, page_size, n_heads, kd, vd, window, scale2, n_splits)
    if (kd <= 96 && vd <= 64) GO(3, 4);
    else if (kd <= 160 && vd <= 128) GO(5, 8);
    else if (kd <= 288 && vd <= 256) GO(9, 16);
    else GO(18, 32);
#undef GO
    GI_CHECK_LAUNCH("latent_attention");
    if (n_splits > 1) {
        latent_merge_kernel<<<(unsigned)(n_rows * n_heads), 64, 0, stream>>>(part, (bf16_t*)out, rows, n_heads, vd, n_splits);
        GI_CHECK_LAUNCH("latent_merge");
    }
    return 0;
}

// The rows of prompts, by the attention plan's tiles ({first row, rows, first position, slot}, of up to tile_rows rows each): heads in
// groups of 16, at most 8 groups (128 heads).
GI_API int gi_latent_attention_tiles_supports(int n_heads, int kd, int vd, int page_size) {
    return gi_latent_attention_supports(kd, vd, page_size) && (n_heads + 15) / 16 <= 8;
}

template <int KS, int DT>
static int allow_latent_tiles_lds() {
    static bool allowed = false;                         // (per instantiation; more than 64 KiB of LDS must be asked for)
    if (!allowed) {
        const size_t lds_bytes = (size_t)(32 * (KS * 32 + 8) + DT * 16 * 40) * 2;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(&latent_attention_tiles_kernel<KS, DT, (KS <= 9)>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess)
            return gi_fail("latent_attention: %zu bytes of LDS are not granted", lds_bytes);
        allowed = true;
    }
    return 0;
}

// Asks for the kernels' LDS once, outside any captured pass (a part calls it when it is built).
GI_API int gi_latent_attention_tiles_prepare() {
    int rc = allow_latent_tiles_lds<3, 4>();
    if (!rc) rc = allow_latent_tiles_lds<5, 8>();
    if (!rc) rc = allow_latent_tiles_lds<9, 16>();
    if (!rc) rc = allow_latent_tiles_lds<18, 32>();
    return rc;
}

template <int KS, int DT>
static int launch_latent_tiles(const void* q, const void* cache, void* out, const void* tiles, int n_tiles, int tile_rows, const int* table, int table_stride,
                               long page_stride, int page_size, int n_heads, int kd, int vd, int window, float scale2, hipStream_t stream) {
    const int HG = (n_heads + 15) / 16, TR = 8 / HG > 0 ? 8 / HG : 1;
    const int pieces = (tile_rows + TR - 1) / TR;
    const size_t lds_bytes = (size_t)(32 * (KS * 32 + 8) + DT * 16 * 40) * 2;
    if (int rc = allow_latent_tiles_lds<KS, DT>()) return rc;
    latent_attention_tiles_kernel<KS, DT, (KS <= 9)><<<(unsigned)(n_tiles * pieces), 64 * TR * HG, lds_bytes, stream>>>(
        (const bf16_t*)q, (const bf16_t*)cache, (bf16_t*)out, (const int4*)tiles, pieces, TR, HG, table, table_stride, page_stride, page_size, n_heads, kd, vd, window, scale2);
    return 0;
}

GI_API int gi_latent_attention_tiles_bf16(const void* q, const void* cache, void* out, const void* tiles, int n_tiles, int tile_rows, const int* table, int table_stride,
                                          long page_stride, int page_size, int n_heads, int kd, int vd, int window, float scale, hipStream_t stream) {
    GI_REQUIRE(n_tiles > 0 && tile_rows > 0 && n_heads > 0 && gi_latent_attention_tiles_supports(n_heads, kd, vd, page_size),
               "latent_attention (tiles): sizes (%d tiles of %d rows, heads %d, keys %d, values %d, pages of %d) are not taken", n_tiles, tile_rows, n_heads, kd, vd, page_size);
    GI_REQUIRE(window >= 0 && page_stride >= (long)page_size * (kd + vd) && page_stride % 8 == 0 && ((uintptr_t)cache & 15) == 0 && ((uintptr_t)q & 15) == 0 &&
               ((uintptr_t)tiles & 15) == 0, "latent_attention (tiles): bad window, page stride or alignment");
    GI_REQUIRE((long)n_tiles * tile_rows < 2147483647L, "latent_attention (tiles): too many rows");
    const float scale2 = scale * 1.4426950408889634f;
    int rc;
#define GO(KS, DT) rc = launch_latent_tiles<KS, DT>(q, cache, out, tiles, n_tiles, tile_rows, table, table_stride, page_stride, page_size, n_heads, kd, vd, window, scale2, stream)
    if (kd <= 96 && vd <= 64) GO(3, 4);
    else if (kd <= 160 && vd <= 128) GO(5, 8);
    else if (kd <= 288 && vd <= 256) GO(9, 16);
    else GO(18, 32);
#undef GO
    if (rc) return rc;
    GI_CHECK_LAUNCH("latent_attention (tiles)");
    return 0;
}
