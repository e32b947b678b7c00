// Recurrent mixers: a step's rows cut into the requests' runs on the device, the matrix memory with exponential gates
// (mLSTM) stepped token by token in 32-bit, and the norm and gate on its heads' outputs.
//
// The matrix memory of one head is S [dk][dv] with a normaliser n [dk] and a running maximum m of the gates' logarithms:
//     m_t = max(f_t + m_(t-1), i_t)
//     S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T        n_t likewise with k_t alone
//     o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
// with i_t = cap * tanh(pre_i / cap) and f_t = logsigmoid(cap * tanh(pre_f / cap)); S, n and m are zero at a sequence's start
// (m = 0, not minus infinity).  Columns of S never meet, and n is the column that S would have for a value that is always 1.
// So one wave owns a "tile" of four columns, three of S and n, for one head of one request, and walks the request's rows of this
// step in order; every tile of a head computes n and m alike and keeps its own copy (a tile that read them from a common place
// would race with the tile that writes them).  State of one request slot: [head][tile]{[dk][4], m, 3 unused}, 32-bit.
//
// Lane = (column, group of rows): a lane keeps ROWS rows (16 apart) of one column in registers; the 16 groups' shares of a
// column's S^T q (neighbouring lanes) are added by the vector unit's lane moves, and n . q, which every column's output is
// divided by, is read from the last column's lane.  A token so costs no barrier and no trip through LDS for the sums, three
// instructions per row of a lane, and the chip gets heads * dv / 3 independent waves: the recurrence is sequential in the
// tokens, so what counts is how few instructions a wave spends on one.
// Per token k and q*scale come through LDS (read as broadcasts).  The k, q and v of a block of tokens are asked for while the
// block before it is worked on and laid into LDS at its end, so that no token waits for memory.  The gates of 64 tokens are made
// at once, lane by token: m runs along them one after the other (an addition and a maximum each), and the exponentials it needs
// are then taken for all 64 at once.  Every sum's order is fixed by dk alone: a request's results have the same bits however
// its rows are cut into steps.
//
// The gated delta rule keeps a memory M [dk][dv] per head.  A token with decay d, step size s, unit key k and query q lets it decay,
// M <- d M, moves what it holds along k towards v, M <- M + k e^T with e = s (v - M^T k), and reads it, y = M^T q: the read-out
// sees the token's own write.  Columns of M never meet here either, so a wave owns four of them, lanes as above; a token costs
// two sums over the key's rows, which the kernel takes in one pass over the memory as it was before the token.  Before the rule,
// q, k and v pass a short causal convolution over the request's rows (the last taps - 1 rows before a step are part of the
// request's state) and SiLU, and q and k are made unit vectors; after it, a head's output is divided by its root mean square, as
// the matrix memory's.
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

// Lane `u`'s value of x, u the same for every lane.
__device__ __forceinline__ float lane_value(float x, int u) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), u)); }

// Sum over each group of RG neighbouring lanes (4, 8 or 16: within a row of 16 lanes), by the data-parallel moves of the vector
// unit: a lane and its mirror image in the group, then lanes two apart, then neighbours.  Every lane of a group ends with the
// same bits (each level adds the same two numbers on both sides).
template <int CTRL>
__device__ __forceinline__ float dpp_moved(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, false));
}
template <int RG>
__device__ __forceinline__ float group_sum(float x) {
    static_assert(RG == 4 || RG == 8 || RG == 16, "groups of 4, 8 or 16 lanes");
    if constexpr (RG == 16) x += dpp_moved<0x140>(x);        // row_mirror: lane i <-> 15 - i
    if constexpr (RG >= 8) x += dpp_moved<0x141>(x);         // row_half_mirror: lane i <-> 7 - i
    x += dpp_moved<0x4E>(x);                                 // quad_perm [2, 3, 0, 1]
    x += dpp_moved<0xB1>(x);                                 // quad_perm [1, 0, 3, 2]
    return x;
}

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <int ROWS>
__global__ __launch_bounds__(64) void mlstm_scan_kernel(const float* __restrict__ proj, long ld, int q_off, int k_off, int v_off, int i_off, int f_off,
                                                       const float* __restrict__ i_bias, const float* __restrict__ f_bias, float cap, float q_scale,
                                                       const int* __restrict__ seg_start, const int* __restrict__ seg_len,
                                                       const int* __restrict__ row_slot, float* __restrict__ state, long state_stride,
                                                       float* __restrict__ out, long ldo, float* __restrict__ den, int dk, int dv) {
    constexpr int C = 4, VC = 3;                 // columns a wave holds: three of S and n (as the column of a value that is always 1)
    constexpr int RG = 64 / C;                   // groups of rows: lane = column * RG + group, so that a column's groups are neighbouring lanes
    constexpr int KQ = RG * ROWS;                // rows a token's k and q cover (dk, padded with zeros)
    constexpr int TB = 1024 / KQ;                // tokens staged at a time: their k, q and v wait in LDS while the block before them is worked on
    constexpr int PER = TB * KQ / 64;            // (k, q) pairs a lane brings per block
    static_assert(TB >= 2 && TB <= 16 && 64 % TB == 0 && TB * VC <= 64, "staging blocks divide the gates' blocks of 64 tokens; a lane brings one value");
    __shared__ float2 kq_s[2][TB][KQ];
    __shared__ float v_s[2][TB][C];
    __shared__ float4 coef[64];                  // per token of the gates' block: {decay of what is held, weight of what comes, exp(-m), -}
    const int seg = blockIdx.x, h = blockIdx.y, vt = blockIdx.z, n_tiles = gridDim.z;
    const int lane = threadIdx.x, c = lane / RG, rg = lane % RG;
    const int n = seg_len[seg];
    if (n <= 0) return;
    const int t0 = seg_start[seg];
    const int col = vt * VC + c;
    const bool live = c < VC && col < dv;
    float* st = state + (size_t)row_slot[t0] * state_stride + ((size_t)h * n_tiles + vt) * ((size_t)dk * C + 4);
    float* st_m = st + (size_t)dk * C;

    float S[ROWS];
#pragma unroll
    for (int rr = 0; rr < ROWS; ++rr) {
        const int i = rr * RG + rg;                  // (a lane's rows lie RG apart: the groups' reads of LDS then fall into different banks)
        S[rr] = i < dk ? st[(size_t)i * C + c] : 0.f;
    }
    float m = st_m[0];
    const float bi = i_bias[h], bf = f_bias[h];

    // A block of TB tokens from `first` on (rows beyond the request's last are read as its last: finite, and never used).
    float2 kq_reg[PER];
    float v_reg;
    auto fetch = [&](int first) {
#pragma unroll
        for (int e = 0; e < PER; ++e) {
            const int idx = lane + 64 * e, u = idx / KQ, i = idx % KQ;
            const float* row = proj + (size_t)(t0 + min(first + u, n - 1)) * ld;
            const int ic = min(i, dk - 1);
            const float kk = row[k_off + h * dk + ic], qq = row[q_off + h * dk + ic] * q_scale;
            kq_reg[e] = i < dk ? float2{kk, qq} : float2{0.f, 0.f};
        }
        const int idx = min(lane, TB * VC - 1), u = idx / VC, cc = min(vt * VC + idx % VC, dv - 1);
        v_reg = proj[(size_t)(t0 + min(first + u, n - 1)) * ld + v_off + h * dv + cc];
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int e = 0; e < PER; ++e) {
            const int idx = lane + 64 * e;
            kq_s[buf][idx / KQ][idx % KQ] = kq_reg[e];
        }
        if (lane < TB * VC) v_s[buf][lane / VC][lane % VC] = v_reg;
    };
    if (lane < 2 * TB) v_s[lane / TB][lane % TB][VC] = 1.0f;          // the value that makes a column of S the normaliser n
    fetch(0);
    stash(0);
    int buf = 0;

    for (int b0 = 0; b0 < n; b0 += 64) {
        const int count = min(64, n - b0);
        // The gates of this block's tokens, lane u token u; then m along the block, one token after the other (two numbers a
        // token: cheap), each lane keeping the m before and after its own token; then the exponentials, all tokens at once.
        const float* g = proj + (size_t)(t0 + b0 + min(lane, count - 1)) * ld;
        const float li = cap * tanhf((g[i_off + h] + bi) / cap);
        const float lf = log_sigmoid(cap * tanhf((g[f_off + h] + bf) / cap));
        float m_before = 0.f, m_after = 0.f;
        for (int u = 0; u < count; ++u) {
            const float m_new = fmaxf(lane_value(lf, u) + m, lane_value(li, u));        // (u is the same for the whole wave)
            if (lane == u) { m_before = m; m_after = m_new; }
            m = m_new;
        }
        __syncthreads();                             // (one wave: orders this block's reads of coef before the writes)
        coef[lane] = float4{expf(lf + m_before - m_after), expf(li - m_after), expf(-m_after), 0.f};
        __syncthreads();
        for (int s0 = 0; s0 < count; s0 += TB, buf ^= 1) {
            const bool more = b0 + s0 + TB < n;
            if (more) fetch(b0 + s0 + TB);
            const int here = min(TB, count - s0);
            // One token: the memory takes it in; the lane's share of its column's S^T q comes back (of n . q in the last column).
            auto token = [&](int u, float& acc, float& floor_) {
                const float4 cf = coef[s0 + u];
                const float a = cf.x, bv = cf.y * v_s[buf][u][c];
                acc = 0.f, floor_ = cf.z;
#pragma unroll
                for (int rr = 0; rr < ROWS; ++rr) {
                    const float2 kq = kq_s[buf][u][rr * RG + rg];
                    S[rr] = fmaf(a, S[rr], kq.x * bv);
                    acc = fmaf(S[rr], kq.y, acc);
                }
            };
            // The groups' shares are added by lane moves; n . q is then in the last column's lanes, the same for the whole wave.
            // The columns' sums leave undivided; what they are to be divided by, max(|n . q|, exp(-m)) + 1e-6, one number per
            // token and head, is written by the head's first tile, and whoever reads the sums divides (the kernel behind this
            // one reads every sum once anyway; a division per token in every wave is a sixth of what a wave does here).
            auto finish = [&](int u, float acc, float floor_) {
                acc = group_sum<RG>(acc);
                const size_t t = (size_t)(t0 + b0 + s0 + u);
                if (rg == 0 && live) out[t * ldo + h * dv + col] = acc;
                if (vt == 0 && lane == VC * RG) den[t * gridDim.y + h] = fmaxf(fabsf(acc), floor_) + 1e-6f;
            };
            constexpr int UB = TB >= 4 ? 4 : TB;     // so many tokens at a time, so that their reads of LDS go out together
            int u = 0;
            for (; u + UB <= here; u += UB) {
                float acc[UB], floor_[UB];
#pragma unroll
                for (int k = 0; k < UB; ++k) token(u + k, acc[k], floor_[k]);
#pragma unroll
                for (int k = 0; k < UB; ++k) finish(u + k, acc[k], floor_[k]);
            }
            for (; u < here; ++u) {
                float acc, floor_;
                token(u, acc, floor_);
                finish(u, acc, floor_);
            }
            __syncthreads();                         // this block's reads are done before the buffer after next is written
            if (more) stash(buf ^ 1);
            __syncthreads();
        }
    }
#pragma unroll
    for (int rr = 0; rr < ROWS; ++rr) {
        const int i = rr * RG + rg;
        if (i < dk && (live || c == VC)) st[(size_t)i * C + c] = S[rr];
    }
    if (lane == 0) st_m[0] = m;
}

// y[t, h*dv + d] = w[h*dv + d] * o[t, h, d] * rsqrt(mean_d(o[t, h, :]^2) + eps) * sigmoid(g[t, h*dv + d]): one wave per (row, head).
// With `den` [rows, heads], o is what the rows hold divided by den[t, h] (the matrix memory's sums and their divisor).
// w_head_stride: dv where every head has weights of its own, 0 where all heads share one [dv]; gate_act 0: sigmoid(g), 1: SiLU, g sigmoid(g).
template <typename TW, typename TO>
__global__ __launch_bounds__(64) void head_norm_gate_kernel(const float* __restrict__ o, long ldo, const float* __restrict__ den,
                                                           const float* __restrict__ g, long ldg, const TW* __restrict__ w,
                                                           TO* __restrict__ y, long ldy, int n_heads, int dv, float eps, int w_head_stride, int gate_act) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float* orow = o + (size_t)t * ldo + (size_t)h * dv;
    const float by = den ? den[(size_t)t * n_heads + h] : 1.0f;
    float ss = 0.f;
    for (int d = lane; d < dv; d += 64) {
        const float v = den ? orow[d] / by : orow[d];
        ss = fmaf(v, v, ss);
    }
    const float r = 1.0f / sqrtf(wave_sum(ss) / (float)dv + eps);
    for (int d = lane; d < dv; d += 64) {
        const float v = den ? orow[d] / by : orow[d];
        const float z = g[(size_t)t * ldg + (size_t)h * dv + d];
        const float gate = (gate_act ? z : 1.0f) / (1.0f + expf(-z));
        store_f32(y, (size_t)t * ldy + (size_t)h * dv + d, load_f32(w, (size_t)h * w_head_stride + d) * (v * r) * gate);
    }
}


// ------------------------------------------------------------------------------------- gated delta rule
constexpr int DELTA_MAX_TAPS = 16;

__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// How many of the rows before row t belong to the same request's run in this step, up to `most`.
__device__ __forceinline__ int rows_before(const int* __restrict__ slot, const int* __restrict__ pos, int t, int most) {
    int r = 0;
    while (r < most && t - r - 1 >= 0 && slot[t - r - 1] == slot[t] && pos[t - r - 1] == pos[t] - r - 1) ++r;
    return r;
}

// What the rule needs of one row, one wave per (row, item).  The convolved columns of `proj` are [conv_off, conv_off + n_conv):
// query heads [n_kv][dk], key heads [n_kv][dk], value heads [n_heads][dv], in this order; `taps` [n_conv][n_taps] float32, the
// last tap the row's own; `tail` [slots][n_taps - 1][n_conv] the request's last rows before this step (zeros at its start).
//   items 0 .. 2 n_kv - 1     a query or key head: convolution, SiLU, divided by sqrt(sum of squares + 1e-6); queries times q_scale
//   items 2 n_kv .. + n_heads a value head: convolution, SiLU
//   the last item             per head the decay exp(-exp(a_log) softplus(pre_a + dt_bias)) and the step size sigmoid(pre_b)
// qkv: float32 [rows, n_conv] in the columns' order; gates: float32 [rows, 2 n_heads], decays then step sizes.
// move_tail: every row of the step is its request's only one (a decode step); the thread that has read a channel's tail then also
// moves it on by the row's own input, and no other kernel needs to (with several rows of a request in a step, rows read the tail
// that others would be writing: `delta_tail_kernel` does it behind this one).
__global__ __launch_bounds__(64) void delta_prepare_kernel(const float* __restrict__ proj, long ld, int conv_off, int a_off, int b_off,
                                                          const float* __restrict__ taps, int n_taps, float* __restrict__ tail, long tail_stride, int move_tail,
                                                          const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                                                          const int* __restrict__ slot, const int* __restrict__ pos, float* __restrict__ qkv,
                                                          float* __restrict__ gates, int n_heads, int n_kv, int dk, int dv, float q_scale) {
    const int t = blockIdx.x, item = blockIdx.y, lane = threadIdx.x;
    if (item == 2 * n_kv + n_heads) {
        for (int h = lane; h < n_heads; h += 64) {
            const float pre_a = proj[(size_t)t * ld + a_off + h], pre_b = proj[(size_t)t * ld + b_off + h];
            gates[(size_t)t * 2 * n_heads + h] = expf(-expf(a_log[h]) * softplus_f(pre_a + dt_bias[h]));
            gates[(size_t)t * 2 * n_heads + n_heads + h] = 1.0f / (1.0f + expf(-pre_b));
        }
        return;
    }
    const int n_conv = 2 * n_kv * dk + n_heads * dv;
    const bool unit = item < 2 * n_kv;
    const int first = unit ? item * dk : 2 * n_kv * dk + (item - 2 * n_kv) * dv, width = unit ? dk : dv;
    const int before = rows_before(slot, pos, t, n_taps - 1);
    float* old = tail + (size_t)slot[t] * tail_stride;
    float ss = 0.f;
    for (int d = lane; d < width; d += 64) {
        const int c = first + d;
        float y = 0.f;
        for (int j = 0; j < n_taps; ++j) {
            const int back = n_taps - 1 - j;                      // rows before t that tap j reads
            const float x = back <= before ? proj[(size_t)(t - back) * ld + conv_off + c] : old[(size_t)(n_taps - 1 - (back - before)) * n_conv + c];
            y = fmaf(taps[(size_t)c * n_taps + j], x, y);
        }
        if (move_tail) {
            for (int i = 0; i + 2 < n_taps; ++i) old[(size_t)i * n_conv + c] = old[(size_t)(i + 1) * n_conv + c];
            if (n_taps > 1) old[(size_t)(n_taps - 2) * n_conv + c] = proj[(size_t)t * ld + conv_off + c];
        }
        y = y / (1.0f + expf(-y));
        qkv[(size_t)t * n_conv + c] = y;                          // (read back below by the lane that wrote it)
        ss = fmaf(y, y, ss);
    }
    if (!unit) return;
    const float r = (item < n_kv ? q_scale : 1.0f) / sqrtf(wave_sum(ss) + 1e-6f);
    for (int d = lane; d < width; d += 64) qkv[(size_t)t * n_conv + first + d] *= r;
}

// After a step's rows the request's tail is its last n_taps - 1 inputs: of this step's rows, and of the old tail where the step
// brought fewer.  One workgroup per request of the step; a thread reads all it needs of a channel before it writes.
__global__ __launch_bounds__(256) void delta_tail_kernel(const float* __restrict__ proj, long ld, int conv_off, int n_conv, int n_taps,
                                                        const int* __restrict__ seg_start, const int* __restrict__ seg_len,
                                                        const int* __restrict__ slot, float* __restrict__ tail, long tail_stride) {
    const int n = seg_len[blockIdx.x];
    if (n <= 0) return;
    const int t0 = seg_start[blockIdx.x], keep = n_taps - 1;
    float* mine = tail + (size_t)slot[t0] * tail_stride;
    for (int c = threadIdx.x; c < n_conv; c += 256) {
        float held[DELTA_MAX_TAPS];
#pragma unroll
        for (int s = 0; s < DELTA_MAX_TAPS; ++s) {
            if (s >= keep) break;
            const int e = n - keep + s;                           // row of the step, or (negative) place before it
            held[s] = e >= 0 ? proj[(size_t)(t0 + e) * ld + conv_off + c] : mine[(size_t)(keep + e) * n_conv + c];
        }
#pragma unroll
        for (int s = 0; s < DELTA_MAX_TAPS; ++s) {
            if (s >= keep) break;
            mine[(size_t)s * n_conv + c] = held[s];
        }
    }
}

// The rule itself: one wave per (request of the step, head, four columns of M).  lane = column * 16 + group of rows; a lane keeps
// the rows 16 apart of its column.  State of a request slot: [head][tile]{[dk][4]}.
// With M the memory before the token, M' = d M + k e^T after it and e = s (v - d M^T k), the read-out is
//     y = M'^T q = d M^T q + e (k . q):
// both sums over the old memory's rows (M^T k and M^T q) and k . q are taken in one pass and reduced side by side, the memory is
// updated behind them, and a token's chain of dependent steps is one pass and one reduction, not two of each.  Every sum over the
// key's rows is the lanes' own shares in a fixed order, then the 16 groups by lane moves: the bits do not depend on the cut.
// Key and query of a block of tokens wait in LDS; the block after it is asked for while this one is worked on.
template <int ROWS>
__global__ __launch_bounds__(64) void delta_scan_kernel(const float* __restrict__ qkv, long ld, const float* __restrict__ gates,
                                                       const int* __restrict__ seg_start, const int* __restrict__ seg_len,
                                                       const int* __restrict__ row_slot, float* __restrict__ state, long state_stride,
                                                       float* __restrict__ out, long ldo, int n_heads, int n_kv, int dk, int dv) {
    constexpr int C = 4, RG = 16, KQ = RG * ROWS;
    constexpr int TB = (1024 / KQ) < 16 ? (1024 / KQ) : 16;      // tokens staged at a time
    constexpr int PER = TB * KQ / 64;            // (k, q) pairs a lane brings per block
    static_assert(TB >= 2 && TB * C <= 64, "a block of 2 to 16 tokens; a lane brings one value and one pair of gates");
    __shared__ float2 kq_s[2][TB][KQ];
    __shared__ float v_s[2][TB][C];
    __shared__ float2 gb_s[2][TB];
    const int seg = blockIdx.x, h = blockIdx.y, vt = blockIdx.z, n_tiles = gridDim.z;
    const int lane = threadIdx.x, c = lane / RG, rg = lane % RG;
    const int n = seg_len[seg];
    if (n <= 0) return;
    const int t0 = seg_start[seg];
    const int col = vt * C + c, kvh = h / (n_heads / n_kv);
    const bool live = col < dv;
    float* st = state + (size_t)row_slot[t0] * state_stride + ((size_t)h * n_tiles + vt) * ((size_t)dk * C);
    const int q_at = kvh * dk, k_at = (n_kv + kvh) * dk, v_at = 2 * n_kv * dk + h * dv;

    float S[ROWS];
#pragma unroll
    for (int rr = 0; rr < ROWS; ++rr) {
        const int i = rr * RG + rg;
        S[rr] = i < dk ? st[(size_t)i * C + c] : 0.f;
    }
    // A block of TB tokens from `first` on (rows beyond the request's last are read as its last: finite, and never used).
    float2 kq_reg[PER], gb_reg;
    float v_reg;
    auto fetch = [&](int first) {
#pragma unroll
        for (int e = 0; e < PER; ++e) {
            const int idx = lane + 64 * e, u = idx / KQ, i = idx % KQ;
            const float* row = qkv + (size_t)(t0 + min(first + u, n - 1)) * ld;
            const int ic = min(i, dk - 1);
            const float kk = row[k_at + ic], qq = row[q_at + ic];
            kq_reg[e] = i < dk ? float2{kk, qq} : float2{0.f, 0.f};
        }
        const int u = min(lane / C, TB - 1), cc = min(vt * C + lane % C, dv - 1);
        v_reg = qkv[(size_t)(t0 + min(first + u, n - 1)) * ld + v_at + cc];
        const float* g = gates + (size_t)(t0 + min(first + min(lane, TB - 1), n - 1)) * 2 * n_heads;
        gb_reg = float2{g[h], g[n_heads + h]};
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int e = 0; e < PER; ++e) {
            const int idx = lane + 64 * e;
            kq_s[buf][idx / KQ][idx % KQ] = kq_reg[e];
        }
        if (lane < TB * C) v_s[buf][lane / C][lane % C] = v_reg;
        if (lane < TB) gb_s[buf][lane] = gb_reg;
    };
    fetch(0);
    stash(0);
    barrier_lds();
    int buf = 0;
    for (int b0 = 0; b0 < n; b0 += TB, buf ^= 1) {
        const int here = min(TB, n - b0);
        const bool more = b0 + TB < n;
        if (more) fetch(b0 + TB);
        for (int u = 0; u < here; ++u) {
            const float2 gb = gb_s[buf][u];
            float kx[ROWS];
            float sk = 0.f, sq = 0.f, kq = 0.f;
#pragma unroll
            for (int rr = 0; rr < ROWS; ++rr) {
                const float2 pair = kq_s[buf][u][rr * RG + rg];
                kx[rr] = pair.x;
                sk = fmaf(S[rr], pair.x, sk);
                sq = fmaf(S[rr], pair.y, sq);
                kq = fmaf(pair.x, pair.y, kq);
            }
            sk = group_sum<RG>(sk);
            sq = group_sum<RG>(sq);
            kq = group_sum<RG>(kq);
            const float w = gb.y * (v_s[buf][u][c] - gb.x * sk);       // s (v - d M^T k)
#pragma unroll
            for (int rr = 0; rr < ROWS; ++rr) S[rr] = fmaf(gb.x, S[rr], kx[rr] * w);
            if (rg == 0 && live) out[(size_t)(t0 + b0 + u) * ldo + h * dv + col] = fmaf(gb.x, sq, w * kq);
        }
        if (more) stash(buf ^ 1);                // (the buffer the block before this one was read from)
        barrier_lds();
    }
#pragma unroll
    for (int rr = 0; rr < ROWS; ++rr) {
        const int i = rr * RG + rg;
        if (i < dk) st[(size_t)i * C + c] = S[rr];
    }
}

}  // namespace

GI_API int gi_segments(const int* slot, const int* pos, int n_rows, int* seg_start, int* seg_len, int n_segs, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_segs > 0 && n_segs <= n_rows, "segments: %d rows in %d runs", n_rows, n_segs);
    segments_kernel<<<1, 64, 0, stream>>>(slot, pos, n_rows, seg_start, seg_len, n_segs);
    GI_CHECK_LAUNCH("segments");
    return 0;
}

// Floats of one request slot's state for `n_heads` heads of dk x dv: per head and tile of three value channels, [dk][4] and m (padded to 4).
GI_API long gi_mlstm_state_floats(int n_heads, int dk, int dv) {
    return (long)n_heads * ((dv + 2) / 3) * ((long)dk * 4 + 4);
}

GI_API int gi_mlstm_max_key_dim() { return 512; }

// proj: float32 [n_rows, ld], whose columns q_off.. hold q [heads*dk], k_off.. k [heads*dk], v_off.. v [heads*dv], i_off.. and
// f_off.. the gates' pre-activations [heads]; out: float32 [n_rows, ldo] gets the heads' sums S^T q [heads*dv], den: float32
// [n_rows, heads] what each head's sums are to be divided by (o = out / den); state: [slots, state_stride].
GI_API int gi_mlstm_scan(const float* proj, long ld, int q_off, int k_off, int v_off, int i_off, int f_off, const float* i_bias, const float* f_bias,
                         float cap, float q_scale, const int* seg_start, const int* seg_len, int n_segs, const int* row_slot, float* state,
                         long state_stride, float* out, long ldo, float* den, int n_heads, int dk, int dv, hipStream_t stream) {
    GI_REQUIRE(den != nullptr, "mlstm_scan: the divisors need a place");
    GI_REQUIRE(n_segs > 0 && n_heads > 0 && dk > 0 && dk <= 512 && dv > 0, "mlstm_scan: bad sizes (runs %d, heads %d, dk %d, dv %d; dk at most 512)", n_segs, n_heads, dk, dv);
    GI_REQUIRE(cap > 0.f && state_stride >= gi_mlstm_state_floats(n_heads, dk, dv) && ldo >= (long)n_heads * dv, "mlstm_scan: bad cap, state stride or output stride");
    const int tiles = (dv + 2) / 3;
    GI_REQUIRE(n_heads <= 65535 && tiles <= 65535, "mlstm_scan: too many heads or value channels");
    dim3 grid(n_segs, n_heads, tiles);
#define GO(R) mlstm_scan_kernel<R><<<grid, 64, 0, stream>>>(proj, ld, q_off, k_off, v_off, i_off, f_off, i_bias, f_bias, cap, q_scale, seg_start, seg_len, \
                                                           row_slot, state, state_stride, out, ldo, den, dk, dv)
    if (dk <= 64) GO(4); else if (dk <= 128) GO(8); else if (dk <= 256) GO(16); else GO(32);
#undef GO
    GI_CHECK_LAUNCH("mlstm_scan");
    return 0;
}

// Floats of one request slot's state of the gated delta rule: the memories, per head and tile of four value channels [dk][4],
// then the convolutions' tail [n_taps - 1][2 n_kv dk + n_heads dv].
GI_API long gi_delta_memory_floats(int n_heads, int dk, int dv) { return (long)n_heads * ((dv + 3) / 4) * ((long)dk * 4); }
GI_API long gi_delta_state_floats(int n_heads, int n_kv, int dk, int dv, int n_taps) {
    return gi_delta_memory_floats(n_heads, dk, dv) + (long)(n_taps - 1) * (2L * n_kv * dk + (long)n_heads * dv);
}
GI_API int gi_delta_max_key_dim() { return 512; }
GI_API int gi_delta_max_taps() { return DELTA_MAX_TAPS; }

// proj: float32 [n_rows, ld]; see delta_prepare_kernel.  state: [slots, state_stride], a slot's memories then its tail.
GI_API int gi_delta_prepare(const float* proj, long ld, int conv_off, int a_off, int b_off, const float* taps, int n_taps, const float* a_log,
                            const float* dt_bias, const int* slot, const int* pos, float* state, long state_stride, float* qkv, float* gates,
                            int n_rows, int n_heads, int n_kv, int dk, int dv, float q_scale, int move_tail, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0 && dk > 0 && dv > 0, "delta_prepare: bad sizes (rows %d, heads %d, kv heads %d, dk %d, dv %d)",
               n_rows, n_heads, n_kv, dk, dv);
    GI_REQUIRE(n_taps >= 1 && n_taps <= DELTA_MAX_TAPS, "delta_prepare: %d taps, 1 to %d are served", n_taps, DELTA_MAX_TAPS);
    const long n_conv = 2L * n_kv * dk + (long)n_heads * dv;
    GI_REQUIRE(conv_off >= 0 && a_off >= 0 && b_off >= 0 && ld >= conv_off + n_conv && ld >= a_off + n_heads && ld >= b_off + n_heads,
               "delta_prepare: the columns named lie outside the rows");
    GI_REQUIRE(state_stride >= gi_delta_state_floats(n_heads, n_kv, dk, dv, n_taps) && 2 * n_kv + n_heads + 1 <= 65535, "delta_prepare: state stride %ld too small, or too many heads", state_stride);
    dim3 grid(n_rows, 2 * n_kv + n_heads + 1);
    delta_prepare_kernel<<<grid, 64, 0, stream>>>(proj, ld, conv_off, a_off, b_off, taps, n_taps, state + gi_delta_memory_floats(n_heads, dk, dv), state_stride, move_tail,
                                                  a_log, dt_bias, slot, pos, qkv, gates, n_heads, n_kv, dk, dv, q_scale);
    GI_CHECK_LAUNCH("delta_prepare");
    return 0;
}

GI_API int gi_delta_tail(const float* proj, long ld, int conv_off, int n_taps, const int* seg_start, const int* seg_len, int n_segs, const int* slot,
                         float* state, long state_stride, int n_heads, int n_kv, int dk, int dv, hipStream_t stream) {
    GI_REQUIRE(n_segs > 0 && n_taps >= 1 && n_taps <= DELTA_MAX_TAPS, "delta_tail: %d runs, %d taps", n_segs, n_taps);
    const long n_conv = 2L * n_kv * dk + (long)n_heads * dv;
    GI_REQUIRE(conv_off >= 0 && ld >= conv_off + n_conv && state_stride >= gi_delta_state_floats(n_heads, n_kv, dk, dv, n_taps), "delta_tail: columns outside the rows, or state stride too small");
    if (n_taps == 1) return 0;
    delta_tail_kernel<<<n_segs, 256, 0, stream>>>(proj, ld, conv_off, (int)n_conv, n_taps, seg_start, seg_len, slot, state + gi_delta_memory_floats(n_heads, dk, dv), state_stride);
    GI_CHECK_LAUNCH("delta_tail");
    return 0;
}

// qkv: float32 [n_rows, ld], a row's unit queries [n_kv][dk], unit keys [n_kv][dk], values [n_heads][dv]; gates: float32 [n_rows, 2 n_heads];
// out: float32 [n_rows, ldo] gets the heads' read-outs [n_heads][dv].
GI_API int gi_delta_scan(const float* qkv, long ld, const float* gates, const int* seg_start, const int* seg_len, int n_segs, const int* row_slot,
                         float* state, long state_stride, float* out, long ldo, int n_heads, int n_kv, int dk, int dv, hipStream_t stream) {
    GI_REQUIRE(n_segs > 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0 && dk > 0 && dk <= 512 && dv > 0, "delta_scan: bad sizes (runs %d, heads %d, kv heads %d, dk %d, dv %d; dk at most 512)",
               n_segs, n_heads, n_kv, dk, dv);
    GI_REQUIRE(ld >= 2L * n_kv * dk + (long)n_heads * dv && ldo >= (long)n_heads * dv && state_stride >= gi_delta_memory_floats(n_heads, dk, dv), "delta_scan: row or state strides too small");
    const int tiles = (dv + 3) / 4;
    GI_REQUIRE(n_heads <= 65535 && tiles <= 65535, "delta_scan: too many heads or value channels");
    dim3 grid(n_segs, n_heads, tiles);
#define GO(R) delta_scan_kernel<R><<<grid, 64, 0, stream>>>(qkv, ld, gates, seg_start, seg_len, row_slot, state, state_stride, out, ldo, n_heads, n_kv, dk, dv)
    if (dk <= 32) GO(2); else if (dk <= 64) GO(4); else if (dk <= 128) GO(8); else if (dk <= 256) GO(16); else GO(32);
#undef GO
    GI_CHECK_LAUNCH("delta_scan");
    return 0;
}

GI_API int gi_head_norm_gate(const float* o, long ldo, const float* den, const float* g, long ldg, const void* w, int w_dtype, void* y, int y_dtype, long ldy, int n_rows,
                             int n_heads, int dv, float eps, int shared_weight, int gate_act, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_heads > 0 && n_heads <= 65535 && dv > 0, "head_norm_gate: bad sizes (rows %d, heads %d, dv %d)", n_rows, n_heads, dv);
    GI_REQUIRE(gate_act == 0 || gate_act == 1, "head_norm_gate: the gate is a sigmoid (0) or SiLU (1)");
    dim3 grid(n_rows, n_heads);
    const int w_head_stride = shared_weight ? 0 : dv;
#define GO(TW, TO) head_norm_gate_kernel<TW, TO><<<grid, 64, 0, stream>>>(o, ldo, den, g, ldg, (const TW*)w, (TO*)y, ldy, n_heads, dv, eps, w_head_stride, gate_act)
    if (w_dtype == GI_F32 && y_dtype == GI_F32) GO(float, float);
    else if (w_dtype == GI_F32 && y_dtype == GI_BF16) GO(float, bf16_t);
    else if (w_dtype == GI_BF16 && y_dtype == GI_BF16) GO(bf16_t, bf16_t);
    else if (w_dtype == GI_BF16 && y_dtype == GI_F32) GO(bf16_t, float);
    else return gi_fail("head_norm_gate: unknown dtypes %d, %d", w_dtype, y_dtype);
#undef GO
    GI_CHECK_LAUNCH("head_norm_gate");
    return 0;
}
