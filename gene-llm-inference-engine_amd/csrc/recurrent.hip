// Recurrent mixers: a step's rows cut into the requests' runs on the device, the matrix memory with exponential gates
// (mLSTM) stepped token by token in 32-bit, and the norm and gate on its heads' outputs.
//
// The matrix memory of one head is S [dk][dv] with a normaliser n [dk] and a running maximum m of the gates' logarithms:
//     m_t = max(f_t + m_(t-1), i_t)
//     S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T        n_t likewise with k_t alone
//     o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
// with i_t = cap * tanh(pre_i / cap) and f_t = logsigmoid(cap * tanh(pre_f / cap)); S, n and m are zero at a sequence's start
// (m = 0, not minus infinity).  Columns of S never meet, so a workgroup owns 64 of them (a "tile") for one head of one
// request and walks the request's rows of this step in order; it keeps its own copy of n and m, which every tile of the head
// computes alike.  State of one request slot: [head][tile]{S tile [dk][64], n [dk, padded to 4], m, 3 unused}, 32-bit.
//
// Inside the workgroup wave r of 4 keeps rows r*ROWS .. r*ROWS+ROWS-1 of the tile in registers, lane j column j.  Per token:
// k and q*scale come through LDS (read as broadcasts), the four waves' shares of S^T q and n . q are added through LDS by
// wave 0, which writes the outputs; the next token's k, q and v are asked for before the current one is worked on.  One
// barrier a token.  The gates of 64 tokens are made at once by wave 0.  Every sum's order is fixed by (dk, ROWS) alone.
#include "common.h"

namespace {

// Rows of a step, in order, are runs of single requests; a run starts where the slot changes or the position does not follow.
__global__ __launch_bounds__(64) void segments_kernel(const int* __restrict__ slot, const int* __restrict__ pos, int n_rows,
                                                     int* __restrict__ seg_start, int* __restrict__ seg_len, int n_segs) {
    const int lane = threadIdx.x;
    int count = 0;
    for (int base = 0; base < n_rows; base += 64) {
        const int t = base + lane;
        const bool first = t < n_rows && (t == 0 || slot[t] != slot[t - 1] || pos[t] != pos[t - 1] + 1);
        const unsigned long long mask = __ballot(first);
        const int idx = count + __popcll(mask & ((1ull << lane) - 1ull));
        if (first && idx < n_segs) seg_start[idx] = t;
        count += __popcll(mask);
    }
    __threadfence_block();
    __syncthreads();
    for (int s = lane; s < n_segs; s += 64) seg_len[s] = s < count ? ((s + 1 < count ? seg_start[s + 1] : n_rows) - seg_start[s]) : 0;
}

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <int ROWS>
__global__ __launch_bounds__(256) void mlstm_scan_kernel(const float* __restrict__ proj, long ld, int q_off, int k_off, int v_off, int i_off, int f_off,
                                                        const float* __restrict__ i_bias, const float* __restrict__ f_bias, float cap, float q_scale,
                                                        const int* __restrict__ seg_start, const int* __restrict__ seg_len,
                                                        const int* __restrict__ row_slot, float* __restrict__ state, long state_stride,
                                                        float* __restrict__ out, long ldo, int dk, int dv) {
    __shared__ float2 kq_s[2][4 * ROWS];
    __shared__ float red[2][4][64];
    __shared__ float red_n[2][4];
    __shared__ float gate_i[64], gate_f[64];
    const int seg = blockIdx.x, h = blockIdx.y, vt = blockIdx.z, n_tiles = gridDim.z;
    const int tid = threadIdx.x, r = tid >> 6, j = tid & 63;
    const int n = seg_len[seg];
    if (n <= 0) return;
    const int t0 = seg_start[seg];
    const int col = vt * 64 + j;
    const bool live = col < dv;
    const int n_pad = (dk + 3) & ~3;
    float* st = state + (size_t)row_slot[t0] * state_stride + ((size_t)h * n_tiles + vt) * ((size_t)dk * 64 + n_pad + 4);
    float* st_n = st + (size_t)dk * 64;
    float* st_m = st_n + n_pad;

    float S[ROWS], nn[ROWS];
    const int row0 = r * ROWS;
#pragma unroll
    for (int rr = 0; rr < ROWS; ++rr) {
        const int i = row0 + rr;
        S[rr] = i < dk ? st[(size_t)i * 64 + j] : 0.f;
        nn[rr] = i < dk ? st_n[i] : 0.f;
    }
    float m = st_m[0];
    const float bi = i_bias[h], bf = f_bias[h];

    // the first token's k and q
    const float* row = proj + (size_t)t0 * ld;
    if (tid < 4 * ROWS) kq_s[0][tid] = tid < dk ? float2{row[k_off + h * dk + tid], row[q_off + h * dk + tid] * q_scale} : float2{0.f, 0.f};
    float v_next = live ? row[v_off + h * dv + col] : 0.f;

    for (int b0 = 0; b0 < n; b0 += 64) {
        const int count = min(64, n - b0);
        if (tid < count) {                           // (wave 0: the gates of this block's tokens)
            const float* g = proj + (size_t)(t0 + b0 + tid) * ld;
            gate_i[tid] = cap * tanhf((g[i_off + h] + bi) / cap);
            gate_f[tid] = log_sigmoid(cap * tanhf((g[f_off + h] + bf) / cap));
        }
        __syncthreads();
        for (int u = 0; u < count; ++u) {
            const int t = t0 + b0 + u, buf = u & 1;
            const bool more = b0 + u + 1 < n;
            const float* next = proj + (size_t)(t + (more ? 1 : 0)) * ld;
            float2 kq_next = {0.f, 0.f};
            if (tid < dk) kq_next = float2{next[k_off + h * dk + tid], next[q_off + h * dk + tid] * q_scale};
            const float v_j = v_next;
            v_next = live ? next[v_off + h * dv + col] : 0.f;

            const float ig = gate_i[u], fg = gate_f[u];
            const float m_new = fmaxf(fg + m, ig);
            const float a = expf(fg + m - m_new), b = expf(ig - m_new);
            m = m_new;
            const float bv = b * v_j;
            float acc = 0.f, nq = 0.f;
#pragma unroll
            for (int rr = 0; rr < ROWS; ++rr) {
                const float2 kq = kq_s[buf][row0 + rr];
                S[rr] = fmaf(a, S[rr], kq.x * bv);
                acc = fmaf(S[rr], kq.y, acc);
                nn[rr] = fmaf(a, nn[rr], b * kq.x);
                nq = fmaf(nn[rr], kq.y, nq);
            }
            red[buf][r][j] = acc;
            if (j == 0) red_n[buf][r] = nq;
            if (tid < 4 * ROWS) kq_s[buf ^ 1][tid] = kq_next;
            __syncthreads();
            if (r == 0 && live) {
                const float num = (red[buf][0][j] + red[buf][1][j]) + (red[buf][2][j] + red[buf][3][j]);
                const float dot = (red_n[buf][0] + red_n[buf][1]) + (red_n[buf][2] + red_n[buf][3]);
                out[(size_t)t * ldo + h * dv + col] = num / (fmaxf(fabsf(dot), expf(-m)) + 1e-6f);
            }
        }
    }
#pragma unroll
    for (int rr = 0; rr < ROWS; ++rr) {
        const int i = row0 + rr;
        if (i < dk) {
            st[(size_t)i * 64 + j] = S[rr];
            if (j == 0) st_n[i] = nn[rr];
        }
    }
    if (tid == 0) st_m[0] = m;
}

// y[t, h*dv + d] = w[h*dv + d] * o[t, h, d] * rsqrt(mean_d(o[t, h, :]^2) + eps) * sigmoid(g[t, h*dv + d]): one wave per (row, head).
template <typename TW, typename TO>
__global__ __launch_bounds__(64) void head_norm_gate_kernel(const float* __restrict__ o, long ldo, const float* __restrict__ g, long ldg,
                                                           const TW* __restrict__ w, TO* __restrict__ y, long ldy, int n_heads, int dv, float eps) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float* orow = o + (size_t)t * ldo + (size_t)h * dv;
    float ss = 0.f;
    for (int d = lane; d < dv; d += 64) ss = fmaf(orow[d], orow[d], ss);
    const float r = 1.0f / sqrtf(wave_sum(ss) / (float)dv + eps);
    for (int d = lane; d < dv; d += 64) {
        const float gate = 1.0f / (1.0f + expf(-g[(size_t)t * ldg + (size_t)h * dv + d]));
        store_f32(y, (size_t)t * ldy + (size_t)h * dv + d, load_f32(w, (size_t)h * dv + d) * (orow[d] * r) * gate);
    }
}

}  // namespace

GI_API int gi_segments(const int* slot, const int* pos, int n_rows, int* seg_start, int* seg_len, int n_segs, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_segs > 0 && n_segs <= n_rows, "segments: %d rows in %d runs", n_rows, n_segs);
    segments_kernel<<<1, 64, 0, stream>>>(slot, pos, n_rows, seg_start, seg_len, n_segs);
    GI_CHECK_LAUNCH("segments");
    return 0;
}

// Floats of one request slot's state for `n_heads` heads of dk x dv.
GI_API long gi_mlstm_state_floats(int n_heads, int dk, int dv) {
    return (long)n_heads * ((dv + 63) / 64) * ((long)dk * 64 + ((dk + 3) & ~3) + 4);
}

GI_API int gi_mlstm_max_key_dim() { return 256; }

// proj: float32 [n_rows, ld], whose columns q_off.. hold q [heads*dk], k_off.. k [heads*dk], v_off.. v [heads*dv], i_off.. and
// f_off.. the gates' pre-activations [heads]; out: float32 [n_rows, ldo] gets o [heads*dv]; state: [slots, state_stride].
GI_API int gi_mlstm_scan(const float* proj, long ld, int q_off, int k_off, int v_off, int i_off, int f_off, const float* i_bias, const float* f_bias,
                         float cap, float q_scale, const int* seg_start, const int* seg_len, int n_segs, const int* row_slot, float* state,
                         long state_stride, float* out, long ldo, int n_heads, int dk, int dv, hipStream_t stream) {
    GI_REQUIRE(n_segs > 0 && n_heads > 0 && dk > 0 && dk <= 256 && dv > 0, "mlstm_scan: bad sizes (runs %d, heads %d, dk %d, dv %d; dk at most 256)", n_segs, n_heads, dk, dv);
    GI_REQUIRE(cap > 0.f && state_stride >= gi_mlstm_state_floats(n_heads, dk, dv) && ldo >= (long)n_heads * dv, "mlstm_scan: bad cap, state stride or output stride");
    const int tiles = (dv + 63) / 64;
    GI_REQUIRE(n_heads <= 65535 && tiles <= 65535, "mlstm_scan: too many heads or value channels");
    dim3 grid(n_segs, n_heads, tiles);
#define GO(R) mlstm_scan_kernel<R><<<grid, 256, 0, stream>>>(proj, ld, q_off, k_off, v_off, i_off, f_off, i_bias, f_bias, cap, q_scale, seg_start, seg_len, \
                                                            row_slot, state, state_stride, out, ldo, dk, dv)
    if (dk <= 32) GO(8); else if (dk <= 64) GO(16); else if (dk <= 128) GO(32); else GO(64);
#undef GO
    GI_CHECK_LAUNCH("mlstm_scan");
    return 0;
}

GI_API int gi_head_norm_gate(const float* o, long ldo, const float* g, long ldg, const void* w, int w_dtype, void* y, int y_dtype, long ldy, int n_rows,
                             int n_heads, int dv, float eps, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_heads > 0 && n_heads <= 65535 && dv > 0, "head_norm_gate: bad sizes (rows %d, heads %d, dv %d)", n_rows, n_heads, dv);
    dim3 grid(n_rows, n_heads);
#define GO(TW, TO) head_norm_gate_kernel<TW, TO><<<grid, 64, 0, stream>>>(o, ldo, g, ldg, (const TW*)w, (TO*)y, ldy, n_heads, dv, eps)
    if (w_dtype == GI_F32 && y_dtype == GI_F32) GO(float, float);
    else if (w_dtype == GI_F32 && y_dtype == GI_BF16) GO(float, bf16_t);
    else if (w_dtype == GI_BF16 && y_dtype == GI_BF16) GO(bf16_t, bf16_t);
    else if (w_dtype == GI_BF16 && y_dtype == GI_F32) GO(bf16_t, float);
    else return gi_fail("head_norm_gate: unknown dtypes %d, %d", w_dtype, y_dtype);
#undef GO
    GI_CHECK_LAUNCH("head_norm_gate");
    return 0;
}
