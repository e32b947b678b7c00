// Attention through latents: what lies between the down projections and the attention kernel.
//
// A layer of this kind projects a row down twice: to a query latent of `q_rank` numbers, and to a key/value latent of `kv_rank`
// numbers with `rot` more that are one rotated key part for all heads.  Both latents are RMS-normed with weights of their own.
// Only the normed key/value latent c and the rotated part are cached: a page holds, per place, one "key" [kv_rank + rot] and
// nothing else, because with the up projections folded into the query (q' = W_uk^T q per head) and into the output
// (o = W_uv sum_j p_j c_j) the latent is key and value at once:
//     score_j = q' . c_j + q_rot . k_rot_j          out = sum_j softmax(score)_j c_j
// The rotation here turns neighbouring channels, the pair (2i, 2i + 1) by pos * f_i.
//
//   latent_prepare   one wave per (row, which): the query latent normed into the rows the up projection reads; the key/value
//                    latent normed and the rotated part turned, both written to the row's place in its page
//   latent_queries   one wave per (row, head): a head's unrotated channels into the rows the folding product reads, its
//                    rotated channels turned and written behind the place where that product puts q'
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
    for (int d = lane; d < n; d += 64) store_f32(dst, d, load_f32(w, d) * (r * src[d]));
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

}  // namespace

// proj: float32 [n_rows, ld] = [query latent (q_rank) | key/value latent (kv_rank) | rotated key part (rot)]; cos, sin: float32
// [n_rows, rot/2]; cq: [n_rows, ldcq] gets the normed query latent; the cache's pages hold [place][kv_rank + rot].
GI_API int gi_latent_prepare(const float* proj, long ld, int q_rank, int kv_rank, int rot, const void* q_norm, const void* kv_norm, int norm_dtype,
                             float eps, const float* cos_t, const float* sin_t, const int* pos, const int* slot, const int* table, int table_stride,
                             void* cq, int cq_dtype, long ldcq, void* cache, int cache_dtype, long page_stride, int page_size, int n_rows,
                             hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && q_rank > 0 && kv_rank > 0 && rot >= 0 && rot % 2 == 0, "latent_prepare: bad sizes (rows %d, latents %d and %d, %d rotated channels)",
               n_rows, q_rank, kv_rank, rot);
    GI_REQUIRE(ld >= (long)q_rank + kv_rank + rot && ldcq >= q_rank && page_size > 0 && page_stride >= (long)page_size * (kv_rank + rot),
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
