// Recurrent mixers with a fixed-size state per request: the token-shift mixes and the per-head
// scan of an RWKV-style time mixing, and the causal convolution, the scan and the grouped norm of a
// state-space mixer.  Everything between the projections is float32: mixes of the decay branch,
// decays, step sizes, states, sums, norms; the element type T only says how the projections'
// results are read and the mixers' outputs written.
//
// A step is a flat batch of requests: request s brings the tokens cu[s] .. cu[s + 1] - 1 and keeps
// its state in row seq_slots[s] of the state tensors.  Every scan walks a request's tokens in
// order with the state in registers, so a token's sums are formed in one order whatever else the
// step holds and however the request's tokens were cut into steps: in float32 the results are
// equal bit for bit.
//
// How a scan is laid out.  A head's state is a matrix [rows i, columns j]; a token multiplies
// every element once or twice and sums over the rows, and the next token cannot start before.
// What bounds a prompt is therefore the time of one token, and that is the state elements a lane
// holds: a wave takes 4 columns and deals the rows to its 16 lanes a column (RPL rows a lane),
// a workgroup of 4 waves takes 16 columns, a head is ceil(columns / 16) workgroups on compute
// units of their own.  The row sums are folded over the 16 lanes by four rotations inside the
// row of lanes (data-parallel primitives, no trip through LDS).  The tokens' operands come
// through LDS sixteen tokens at a time, the next sixteen travelling from memory meanwhile.  The
// state is kept column-major ([j][i]) so that a lane's rows are contiguous.
#include "common.h"

namespace recurrent {

// the request a token of the flat batch belongs to: the last s with cu[s] <= t
__device__ inline int request_of(const int* __restrict__ cu, int num_seqs, int t) {
    int lo = 0, hi = num_seqs - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (cu[mid] <= t)
            lo = mid;
        else
            hi = mid - 1;
    }
    return lo;
}

__device__ inline float silu(float z) { return z / (1.f + expf(-z)); }

// --------------------------------------------------------------------------- //
// Token shift.  With h' the previous token's row (the request's state row before its first token
// of the step), branch b reads h + (h' - h) * mu[b].  Branches 0..3 are written in the compute
// type, side by side as [4][tokens][width]; branch 4 (the decay's) in float32.
// The state row is replaced by the request's last row in a second launch, after every read; in a
// step of single tokens (`single`) a token's workgroup is the only one that touches its request's
// row and replaces it itself.
// --------------------------------------------------------------------------- //
template <typename T>
struct alignas(sizeof(T) * 4) Quad {
    T v[4];
};

template <typename T>
__global__ __launch_bounds__(256) void token_shift_kernel(const T* __restrict__ x, const float* __restrict__ mu,
                                                          float* __restrict__ state, T* __restrict__ mixes,
                                                          float* __restrict__ mix_w, const int* __restrict__ cu,
                                                          const int* __restrict__ seq_slots, int num_seqs,
                                                          int tokens, int width, int single) {
    const int t = blockIdx.x;
    const int s = single ? t : request_of(cu, num_seqs, t);
    const bool first = single || t == cu[s];
    float* prev_state = state + (size_t)seq_slots[s] * width;
    const T* row = x + (size_t)t * width;
    const T* before = x + (size_t)(first ? t : t - 1) * width;
    const size_t plane = (size_t)tokens * width;
    if (width % 4 == 0) {
        // four channels a thread, every access 8 or 16 bytes; the loads of two rounds are asked for together
#pragma unroll 2
        for (int i = 4 * threadIdx.x; i < width; i += 4 * blockDim.x) {
            const Quad<T> hq = *reinterpret_cast<const Quad<T>*>(row + i);
            float p[4];
            if (first) {
                const float4 ps = *reinterpret_cast<const float4*>(prev_state + i);
                p[0] = ps.x; p[1] = ps.y; p[2] = ps.z; p[3] = ps.w;
            } else {
                const Quad<T> pq = *reinterpret_cast<const Quad<T>*>(before + i);
#pragma unroll
                for (int e = 0; e < 4; ++e) p[e] = to_float(pq.v[e]);
            }
            float h[4], d[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                h[e] = to_float(hq.v[e]);
                d[e] = p[e] - h[e];
            }
#pragma unroll
            for (int b = 0; b < 5; ++b) {
                const float4 m = *reinterpret_cast<const float4*>(mu + (size_t)b * width + i);
                const float y[4] = {fmaf(d[0], m.x, h[0]), fmaf(d[1], m.y, h[1]), fmaf(d[2], m.z, h[2]),
                                    fmaf(d[3], m.w, h[3])};
                if (b < 4) {
                    Quad<T> o;
#pragma unroll
                    for (int e = 0; e < 4; ++e) o.v[e] = from_float<T>(y[e]);
                    *reinterpret_cast<Quad<T>*>(mixes + b * plane + (size_t)t * width + i) = o;
                } else {
                    *reinterpret_cast<float4*>(mix_w + (size_t)t * width + i) = make_float4(y[0], y[1], y[2], y[3]);
                }
            }
            if (single) *reinterpret_cast<float4*>(prev_state + i) = make_float4(h[0], h[1], h[2], h[3]);
        }
        return;
    }
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float h = to_float(row[i]);
        const float p = first ? prev_state[i] : to_float(before[i]);
        const float d = p - h;
#pragma unroll
        for (int b = 0; b < 4; ++b)
            mixes[b * plane + (size_t)t * width + i] = from_float<T>(fmaf(d, mu[(size_t)b * width + i], h));
        mix_w[(size_t)t * width + i] = fmaf(d, mu[(size_t)4 * width + i], h);
        if (single) prev_state[i] = h;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void shift_state_kernel(const T* __restrict__ x, float* __restrict__ state,
                                                          const int* __restrict__ cu,
                                                          const int* __restrict__ seq_slots, int width) {
    const int s = blockIdx.x;
    const T* last = x + (size_t)(cu[s + 1] - 1) * width;
    float* dst = state + (size_t)seq_slots[s] * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = to_float(last[i]);
}

// --------------------------------------------------------------------------- //
// Helpers of the scans: the sum over a row of 16 lanes by rotations (every lane gets it; the
// order of the additions is fixed by the lane), and the block of tokens staged in LDS.
// --------------------------------------------------------------------------- //
template <int CTRL>
__device__ inline float ror_add(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true);
    return v + __int_as_float(moved);
}
__device__ inline float row16_sum(float v) {
    v = ror_add<0x128>(v);  // row_ror:8
    v = ror_add<0x124>(v);  // row_ror:4
    v = ror_add<0x122>(v);  // row_ror:2
    v = ror_add<0x121>(v);  // row_ror:1
    return v;
}
// the same sums for N values at once, one rotation of all of them after the other: a value's four
// additions depend on each other, those of different values do not, and a wave that runs alone on
// its SIMD has nothing else to put between dependent instructions
template <int N>
__device__ inline void row16_sums(float (&v)[N]) {
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = ror_add<0x128>(v[i]);
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = ror_add<0x124>(v[i]);
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = ror_add<0x122>(v[i]);
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = ror_add<0x121>(v[i]);
}

// A lane's RPL consecutive state rows from or to memory: sixteen bytes at a time where the rows
// of a column are a multiple of four (a group of four is then wholly inside the column or wholly
// beyond it), else one by one.
template <int RPL>
__device__ inline void state_rows_load(const float* __restrict__ column, int first, int rows, bool live,
                                       float (&state)[RPL]) {
    if constexpr (RPL % 4 == 0) {
        if (rows % 4 == 0) {
#pragma unroll
            for (int q = 0; q < RPL; q += 4) {
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (live && first + q < rows) v = *reinterpret_cast<const float4*>(column + first + q);
                state[q] = v.x; state[q + 1] = v.y; state[q + 2] = v.z; state[q + 3] = v.w;
            }
            return;
        }
    }
#pragma unroll
    for (int ii = 0; ii < RPL; ++ii) state[ii] = (live && first + ii < rows) ? column[first + ii] : 0.f;
}
template <int RPL>
__device__ inline void state_rows_store(float* __restrict__ column, int first, int rows, bool live,
                                        const float (&state)[RPL]) {
    if (!live) return;
    if constexpr (RPL % 4 == 0) {
        if (rows % 4 == 0) {
#pragma unroll
            for (int q = 0; q < RPL; q += 4)
                if (first + q < rows)
                    *reinterpret_cast<float4*>(column + first + q) =
                        make_float4(state[q], state[q + 1], state[q + 2], state[q + 3]);
            return;
        }
    }
#pragma unroll
    for (int ii = 0; ii < RPL; ++ii)
        if (first + ii < rows) column[first + ii] = state[ii];
}

constexpr int SCAN_TOKENS = 16;   // tokens staged at a time
constexpr int SCAN_WAVES = 4;                      // waves of a workgroup
constexpr int SCAN_THREADS = 64 * SCAN_WAVES;
constexpr int SCAN_COLS = 4 * SCAN_WAVES;          // columns of a workgroup: 4 a wave

// --------------------------------------------------------------------------- //
// The time-mixing scan.  Per head, state S[key channel i][value channel j], kept as [j][i].  For a
// token with r, k, v (d each), the decay w_i = exp(-exp(pre_i + bias_i)), formed as a block of
// tokens is fetched, and the bonus u_i:
//   o_j = sum_i r_i (S_ij + u_i k_i v_j)        S_ij <- w_i S_ij + k_i v_j
// o goes out unfinished (float32); wkv_finish_kernel divides every head by its root mean square
// and applies the norm's weight and silu(g).
// --------------------------------------------------------------------------- //
// one state element's share of a token (the same instructions wherever a token is computed)
__device__ inline void wkv_row(float r, float k, float w, float u, float vj, float& state, float& o) {
    const float kv = k * vj;
    o = fmaf(r, fmaf(u, kv, state), o);
    state = fmaf(w, state, kv);
}
__device__ inline float wkv_decay(float pre, float bias) { return expf(-expf(pre + bias)); }

template <typename T, int RPL>
__global__ __launch_bounds__(SCAN_THREADS) __attribute__((amdgpu_waves_per_eu(1, 2))) void wkv_scan_kernel(
    const T* __restrict__ r, const T* __restrict__ k, const T* __restrict__ v, const float* __restrict__ decay_pre,
    const float* __restrict__ decay_bias, const float* __restrict__ bonus, float* __restrict__ raw,
    const int* __restrict__ cu,
    const int* __restrict__ seq_slots, float* __restrict__ S, int heads, int d) {
    constexpr int DP = 16 * RPL;  // rows, padded
    constexpr int PER_THREAD = SCAN_TOKENS * DP / SCAN_THREADS;  // = RPL
    const int s = blockIdx.x, h = blockIdx.y;
    const int t0 = cu[s], t1 = cu[s + 1];
    const int inner = heads * d;
    const int lane = threadIdx.x & (RL_WAVE - 1), wave = threadIdx.x / RL_WAVE;
    const int c = lane & 15;                                  // which share of the rows
    const int col = wave * 4 + (lane >> 4);                   // column of the workgroup
    const int j = blockIdx.z * SCAN_COLS + col;
    const bool live = j < d;
    __shared__ __attribute__((aligned(16))) float sr[SCAN_TOKENS][DP], sk[SCAN_TOKENS][DP], sw[SCAN_TOKENS][DP];
    __shared__ float sv[SCAN_TOKENS][SCAN_COLS];
    float* Sp = S + (((size_t)seq_slots[s] * heads + h) * d + (live ? j : 0)) * d;
    float state[RPL], u[RPL];
    state_rows_load<RPL>(Sp, c * RPL, d, live, state);
#pragma unroll
    for (int ii = 0; ii < RPL; ++ii) {
        const int i = c * RPL + ii;
        u[ii] = i < d ? bonus[h * d + i] : 0.f;
    }
    // A block of tokens from memory into registers, as it lies there: element e of the block's
    // [token][row] arrays.  Nothing is computed from what was asked for until the block is staged
    // (a conversion or an exponential here would wait for the loads where they are issued, and
    // the block before would be computed behind that wait instead of during it).
    T pr[PER_THREAD], pk[PER_THREAD], pv;
    float pw[PER_THREAD], pb[PER_THREAD];
#pragma unroll
    for (int e = 0; e < PER_THREAD; ++e) {
        const int i = (e * SCAN_THREADS + threadIdx.x) % DP;
        pb[e] = i < d ? decay_bias[h * d + i] : 0.f;
    }
    const T zero = from_float<T>(0.f);
    auto fetch = [&](int tb) {
#pragma unroll
        for (int e = 0; e < PER_THREAD; ++e) {
            const int idx = e * SCAN_THREADS + threadIdx.x;
            const int tt = idx / DP, i = idx % DP;
            const bool ok = tb + tt < t1 && i < d;
            const size_t at = (size_t)(tb + tt) * inner + h * d + i;
            pr[e] = ok ? r[at] : zero;
            pk[e] = ok ? k[at] : zero;
            pw[e] = ok ? decay_pre[at] : INFINITY;  // a decay of exactly 0
        }
        // (threads beyond tokens x columns, where a workgroup has more, carry nothing)
        const int tt = threadIdx.x / SCAN_COLS, jj = blockIdx.z * SCAN_COLS + threadIdx.x % SCAN_COLS;
        pv = (tt < SCAN_TOKENS && tb + tt < t1 && jj < d) ? v[(size_t)(tb + tt) * inner + h * d + jj] : zero;
    };
    auto stage = [&]() {
#pragma unroll
        for (int e = 0; e < PER_THREAD; ++e) {
            const int idx = e * SCAN_THREADS + threadIdx.x;
            (&sr[0][0])[idx] = to_float(pr[e]);
            (&sk[0][0])[idx] = to_float(pk[e]);
            (&sw[0][0])[idx] = wkv_decay(pw[e], pb[e]);
        }
        if (threadIdx.x < SCAN_TOKENS * SCAN_COLS) (&sv[0][0])[threadIdx.x] = to_float(pv);
    };
    fetch(t0);
    for (int tb = t0; tb < t1; tb += SCAN_TOKENS) {
        __syncthreads();  // the block before has been read by every wave
        stage();
        __syncthreads();
        if (tb + SCAN_TOKENS < t1) fetch(tb + SCAN_TOKENS);
        const int nt = min(SCAN_TOKENS, t1 - tb);
        auto token = [&](int tt) -> float {  // this lane's rows' share of the token's output
            const float vj = sv[tt][col];
            float o = 0.f;
#pragma unroll
            for (int ii = 0; ii < RPL; ++ii)
                wkv_row(sr[tt][c * RPL + ii], sk[tt][c * RPL + ii], sw[tt][c * RPL + ii], u[ii], vj, state[ii], o);
            return o;
        };
        float* dst = raw + (size_t)tb * inner + h * d + j;
        if (nt == SCAN_TOKENS) {
            // a whole block, unrolled and without a branch between its tokens: the reads of later
            // tokens stand in front of the sums of earlier ones, the lane folds of neighbouring
            // tokens interleave, and only the state's own chain orders the tokens; the block's
            // outputs are stored behind it
            float os[SCAN_TOKENS];
#pragma unroll
            for (int tt = 0; tt < SCAN_TOKENS; ++tt) os[tt] = token(tt);
            row16_sums(os);
            // every lane of a column holds all sixteen sums: lane c stores token c's
            float mine = os[0];
#pragma unroll
            for (int tt = 1; tt < SCAN_TOKENS; ++tt) mine = c == tt ? os[tt] : mine;
            if (live) dst[(size_t)c * inner] = mine;
        } else {
            for (int tt = 0; tt < nt; ++tt) {
                const float o = row16_sum(token(tt));
                if (c == 0 && live) dst[(size_t)tt * inner] = o;
            }
        }
    }
    state_rows_store<RPL>(Sp, c * RPL, d, live, state);
}

// out[t, head] = raw / sqrt(mean(raw^2) + eps) * norm_w * silu(g): one wave a (token, head)
template <typename T>
__global__ __launch_bounds__(256) void wkv_finish_kernel(const float* __restrict__ raw, const T* __restrict__ g,
                                                         const float* __restrict__ norm_w, T* __restrict__ out,
                                                         int rows, int heads, int d, float eps) {
    const int row = blockIdx.x * 4 + threadIdx.x / RL_WAVE;  // (token, head)
    const int lane = threadIdx.x & (RL_WAVE - 1);
    if (row >= rows) return;  // whole waves leave
    const size_t base = (size_t)row * d;
    const int h = row % heads;
    float ss = 0.f;
    for (int i = lane; i < d; i += RL_WAVE) {
        const float o = raw[base + i];
        ss += o * o;
    }
    const float rr = rsqrtf(wave_sum(ss) / (float)d + eps);
    for (int i = lane; i < d; i += RL_WAVE)
        out[base + i] = from_float<T>(raw[base + i] * rr * norm_w[h * d + i] * silu(to_float(g[base + i])));
}

// --------------------------------------------------------------------------- //
// Causal convolution per channel over the columns [col0, col0 + channels) of the packed rows, with
// bias and silu: y_t = silu(b + sum_tap w[c][tap] in(t - (taps - 1) + tap)), where inputs before
// the request's first token of the step come from its state rows (the last taps - 1 inputs it has
// seen, oldest first; zeros when the request begins).  A second launch then shifts the state; in a
// step of single tokens (`single`) the thread of a channel shifts its request's rows itself.
// --------------------------------------------------------------------------- //
#define RL_CONV_MAX_TAPS 16

constexpr int CONV_TOKENS = 8;  // consecutive tokens of the flat batch a workgroup takes in a step with portions

template <typename T>
__global__ __launch_bounds__(256) void causal_conv_kernel(const T* __restrict__ packed, int row_width, int col0,
                                                          const float* __restrict__ w, const float* __restrict__ bias,
                                                          float* __restrict__ state, float* __restrict__ out,
                                                          const int* __restrict__ cu,
                                                          const int* __restrict__ seq_slots, int num_seqs, int tokens,
                                                          int channels, int taps, int single, int per_group) {
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const int held = taps - 1;
    float wt[RL_CONV_MAX_TAPS];  // this channel's taps
#pragma unroll
    for (int tap = 0; tap < RL_CONV_MAX_TAPS; ++tap) wt[tap] = tap < taps ? w[(size_t)c * taps + tap] : 0.f;
    const float b = bias[c];
    const int first = blockIdx.x * per_group;
    int s = single ? first : request_of(cu, num_seqs, first);
    for (int t = first; t < min(tokens, first + per_group); ++t) {
        if (single)
            s = t;
        else
            while (t >= cu[s + 1]) ++s;  // tokens ascend through the requests
        const int offset = single ? 0 : t - cu[s];  // tokens of the request's portion before this one
        float* st = state + (size_t)seq_slots[s] * max(held, 1) * channels;
        float acc = b;
#pragma unroll
        for (int tap = 0; tap < RL_CONV_MAX_TAPS; ++tap) {
            if (tap < taps) {
                const int rel = offset - held + tap;  // offset in the portion of the input this tap meets
                const float in = rel >= 0 ? to_float(packed[(size_t)(t - offset + rel) * row_width + col0 + c])
                                          : st[(size_t)(held + rel) * channels + c];
                acc = fmaf(wt[tap], in, acc);
            }
        }
        out[(size_t)t * channels + c] = silu(acc);
        if (single && held > 0) {
            for (int q = 0; q + 1 < held; ++q) st[(size_t)q * channels + c] = st[(size_t)(q + 1) * channels + c];
            st[(size_t)(held - 1) * channels + c] = to_float(packed[(size_t)t * row_width + col0 + c]);
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void conv_state_kernel(const T* __restrict__ packed, int row_width, int col0,
                                                         float* __restrict__ state, const int* __restrict__ cu,
                                                         const int* __restrict__ seq_slots, int channels, int taps) {
    const int s = blockIdx.x;
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    const int held = taps - 1;
    if (c >= channels || held < 1) return;
    const int t0 = cu[s], n = cu[s + 1] - cu[s];
    float* st = state + (size_t)seq_slots[s] * held * channels;
    float old[RL_CONV_MAX_TAPS];
#pragma unroll
    for (int q = 0; q < RL_CONV_MAX_TAPS; ++q) old[q] = q < held ? st[(size_t)q * channels + c] : 0.f;
#pragma unroll
    for (int q = 0; q < RL_CONV_MAX_TAPS; ++q) {
        if (q >= held) continue;
        const int rel = n - held + q;
        float value = 0.f;
        if (rel >= 0) {
            value = to_float(packed[(size_t)(t0 + rel) * row_width + col0 + c]);
        } else {
#pragma unroll
            for (int z = 0; z < RL_CONV_MAX_TAPS; ++z)
                if (z == q + n) value = old[z];
        }
        st[(size_t)q * channels + c] = value;
    }
}

// --------------------------------------------------------------------------- //
// The state-space scan.  `mixed` rows are [x: heads * P | B: groups * N | C: groups * N] (float32,
// behind convolution and silu); per head, state S[n][p], kept as [p][n].  As a block of tokens is
// fetched the raw step sizes become dt = softplus(dt_raw + dt_bias) and a = exp(-exp(A_log) dt); then
//   S_np <- a S_np + dt B_n x_p          y_p = sum_n S_np C_n + D x_p
// and y_p silu(z_p) is written (z: the first heads * P columns of the packed rows).
// --------------------------------------------------------------------------- //
__device__ inline float ssm_step_size(float raw, float bias) {
    const float pre = raw + bias;
    return pre > 20.f ? pre : log1pf(expf(pre));
}
__device__ inline float ssm_decay(float a_log, float dt) { return expf(-expf(a_log) * dt); }
// one state element's share of a token, and the finished output of a channel
__device__ inline void ssm_row(float a, float B, float C, float dx, float& state, float& y) {
    state = fmaf(B, dx, a * state);
    y = fmaf(state, C, y);
}
__device__ inline float ssm_out(float y, float D, float x, float z) { return fmaf(D, x, y) * silu(z); }

template <typename T, int RPL>
__global__ __launch_bounds__(SCAN_THREADS) __attribute__((amdgpu_waves_per_eu(1, 2))) void ssm_scan_kernel(
    const float* __restrict__ mixed, const float* __restrict__ dt_raw, const float* __restrict__ dt_bias,
    const float* __restrict__ a_log, const float* __restrict__ skip, const T* __restrict__ packed, int row_width, float* __restrict__ out, const int* __restrict__ cu,
    const int* __restrict__ seq_slots, float* __restrict__ S, int heads, int P, int N, int groups) {
    constexpr int NP = 16 * RPL;  // state rows, padded
    constexpr int PER_THREAD = SCAN_TOKENS * NP / SCAN_THREADS;  // = RPL
    const int s = blockIdx.x, h = blockIdx.y;
    const int t0 = cu[s], t1 = cu[s + 1];
    const int inner = heads * P;
    const int channels = inner + 2 * groups * N;
    const int grp = h / (heads / groups);
    const int lane = threadIdx.x & (RL_WAVE - 1), wave = threadIdx.x / RL_WAVE;
    const int c = lane & 15;
    const int col = wave * 4 + (lane >> 4);
    const int p = blockIdx.z * SCAN_COLS + col;
    const bool live = p < P;
    __shared__ __attribute__((aligned(16))) float sB[SCAN_TOKENS][NP], sC[SCAN_TOKENS][NP];
    __shared__ float sx[SCAN_TOKENS][SCAN_COLS], sz[SCAN_TOKENS][SCAN_COLS], sdt[SCAN_TOKENS], sa[SCAN_TOKENS];
    float* Sp = S + (((size_t)seq_slots[s] * heads + h) * P + (live ? p : 0)) * N;
    float state[RPL];
    state_rows_load<RPL>(Sp, c * RPL, N, live, state);
    const float D = skip[h];
    // a block of tokens from memory into registers as it lies there; step sizes and decays are
    // formed when the block is staged, not where its loads are issued
    float pB[PER_THREAD], pC[PER_THREAD], px = 0.f, pd = 0.f;
    T pz = from_float<T>(0.f);
    const float step_bias = dt_bias[h], rate_log = a_log[h];
    auto fetch = [&](int tb) {
#pragma unroll
        for (int e = 0; e < PER_THREAD; ++e) {
            const int idx = e * SCAN_THREADS + threadIdx.x;
            const int tt = idx / NP, n = idx % NP;
            const bool ok = tb + tt < t1 && n < N;
            const float* row = mixed + (size_t)(tb + tt) * channels + inner + grp * N + n;
            pB[e] = ok ? row[0] : 0.f;
            pC[e] = ok ? row[groups * N] : 0.f;
        }
        const int tt = threadIdx.x / SCAN_COLS, pp = blockIdx.z * SCAN_COLS + threadIdx.x % SCAN_COLS;
        const bool ok = tt < SCAN_TOKENS && tb + tt < t1 && pp < P;
        px = ok ? mixed[(size_t)(tb + tt) * channels + h * P + pp] : 0.f;
        pz = ok ? packed[(size_t)(tb + tt) * row_width + h * P + pp] : from_float<T>(0.f);
        // threads 0..15 carry the step sizes, threads 16..31 the decays of the block's tokens
        const int tk = threadIdx.x & 15;
        pd = (threadIdx.x < 32 && tb + tk < t1) ? dt_raw[(size_t)(tb + tk) * heads + h] : 0.f;
    };
    auto stage = [&]() {
#pragma unroll
        for (int e = 0; e < PER_THREAD; ++e) {
            const int idx = e * SCAN_THREADS + threadIdx.x;
            (&sB[0][0])[idx] = pB[e];
            (&sC[0][0])[idx] = pC[e];
        }
        if (threadIdx.x < SCAN_TOKENS * SCAN_COLS) {
            (&sx[0][0])[threadIdx.x] = px;
            (&sz[0][0])[threadIdx.x] = to_float(pz);
        }
        if (threadIdx.x < 32) {
            const float dt = ssm_step_size(pd, step_bias);
            if (threadIdx.x < 16) sdt[threadIdx.x] = dt;
            else sa[threadIdx.x - 16] = ssm_decay(rate_log, dt);
        }
    };
    fetch(t0);
    for (int tb = t0; tb < t1; tb += SCAN_TOKENS) {
        __syncthreads();  // the block before has been read by every wave
        stage();
        __syncthreads();
        if (tb + SCAN_TOKENS < t1) fetch(tb + SCAN_TOKENS);
        const int nt = min(SCAN_TOKENS, t1 - tb);
        auto token = [&](int tt) -> float {
            const float x = sx[tt][col], a = sa[tt];
            const float dx = sdt[tt] * x;
            float y = 0.f;
#pragma unroll
            for (int ii = 0; ii < RPL; ++ii)
                ssm_row(a, sB[tt][c * RPL + ii], sC[tt][c * RPL + ii], dx, state[ii], y);
            return y;  // this lane's rows' share
        };
        float* dst = out + (size_t)tb * inner + h * P + p;
        if (nt == SCAN_TOKENS) {
            // a whole block without a branch between its tokens
            float ys[SCAN_TOKENS];
#pragma unroll
            for (int tt = 0; tt < SCAN_TOKENS; ++tt) ys[tt] = token(tt);
            row16_sums(ys);
            // every lane of a column holds all sixteen sums: lane c finishes and stores token c's
            // (skip term, gate with its exponential and division: once a lane, not once a token)
            float mine = ys[0];
#pragma unroll
            for (int tt = 1; tt < SCAN_TOKENS; ++tt) mine = c == tt ? ys[tt] : mine;
            if (live) dst[(size_t)c * inner] = ssm_out(mine, D, sx[c][col], sz[c][col]);
        } else {
            for (int tt = 0; tt < nt; ++tt) {
                const float y = row16_sum(token(tt));
                if (c == 0 && live) dst[(size_t)tt * inner] = ssm_out(y, D, sx[tt][col], sz[tt][col]);
            }
        }
    }
    state_rows_store<RPL>(Sp, c * RPL, N, live, state);
}

// out[t, part] = y[t, part] / sqrt(mean(y[t, part]^2) + eps) * w, a row in `parts` equal parts
template <typename T>
__global__ __launch_bounds__(256) void group_rmsnorm_kernel(const float* __restrict__ y, const float* __restrict__ w,
                                                            T* __restrict__ out, int width, int parts, float eps) {
    __shared__ float scratch[16];
    const int size = width / parts;
    const size_t base = (size_t)blockIdx.x * width + (size_t)blockIdx.y * size;
    float ss = 0.f;
    for (int i = threadIdx.x; i < size; i += blockDim.x) {
        const float v = y[base + i];
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float rr = rsqrtf(ss / (float)size + eps);
    for (int i = threadIdx.x; i < size; i += blockDim.x)
        out[base + i] = from_float<T>(y[base + i] * rr * w[blockIdx.y * size + i]);
}

}  // namespace recurrent

extern "C" int rl_recurrent_max_head_dim() { return 256; }
extern "C" int rl_conv_max_taps() { return RL_CONV_MAX_TAPS; }

extern "C" int rl_token_shift(const void* x, const float* mu, float* state, void* mixes, float* mix_w,
                              const int* cu, const int* seq_slots, int num_seqs, int tokens, int width,
                              int act_type, hipStream_t stream) {
    if (tokens <= 0 || num_seqs <= 0) return RL_OK;
    if (width < 1) return RL_ERR_ARG;
    const int single = tokens == num_seqs;  // every request brings one token
    if (act_type == RL_F32) {
        hipLaunchKernelGGL(recurrent::token_shift_kernel<float>, dim3(tokens), dim3(256), 0, stream, (const float*)x,
                           mu, state, (float*)mixes, mix_w, cu, seq_slots, num_seqs, tokens, width, single);
        if (!single)
            hipLaunchKernelGGL(recurrent::shift_state_kernel<float>, dim3(num_seqs), dim3(256), 0, stream,
                           (const float*)x, state, cu, seq_slots, width);
    } else if (act_type == RL_BF16) {
        hipLaunchKernelGGL(recurrent::token_shift_kernel<bf16_t>, dim3(tokens), dim3(256), 0, stream,
                           (const bf16_t*)x, mu, state, (bf16_t*)mixes, mix_w, cu, seq_slots, num_seqs, tokens,
                           width, single);
        if (!single)
            hipLaunchKernelGGL(recurrent::shift_state_kernel<bf16_t>, dim3(num_seqs), dim3(256), 0, stream,
                           (const bf16_t*)x, state, cu, seq_slots, width);
    } else {
        return RL_ERR_ARG;
    }
    return rl_launch_status();
}

template <typename T>
static int launch_wkv(const T* r, const T* k, const T* v, const T* g, const float* decay, const float* decay_bias,
                      const float* bonus, const float* norm_w, T* out, float* raw, const int* cu,
                      const int* seq_slots, float* S, int num_seqs, int tokens, int heads, int d, float eps,
                      hipStream_t stream) {
    dim3 grid(num_seqs, heads, (d + recurrent::SCAN_COLS - 1) / recurrent::SCAN_COLS);
#define RL_WKV(RPL)                                                                                              \
    hipLaunchKernelGGL((recurrent::wkv_scan_kernel<T, RPL>), grid, dim3(recurrent::SCAN_THREADS), 0, stream, r, k, v, \
                       decay, decay_bias, bonus, raw, cu, seq_slots, S, heads, d)
    const int rows = (d + 15) / 16;
    if (rows <= 1)
        RL_WKV(1);
    else if (rows <= 2)
        RL_WKV(2);
    else if (rows <= 4)
        RL_WKV(4);
    else if (rows <= 8)
        RL_WKV(8);
    else
        RL_WKV(16);
#undef RL_WKV
    const int heads_rows = tokens * heads;
    hipLaunchKernelGGL(recurrent::wkv_finish_kernel<T>, dim3((heads_rows + 3) / 4), dim3(256), 0, stream, raw, g,
                       norm_w, out, heads_rows, heads, d, eps);
    return rl_launch_status();
}

// decay: the decays' pre-activations [tokens, heads * d]; raw: [tokens, heads * d] float32 scratch
// for the unfinished outputs
extern "C" int rl_wkv_scan(const void* r, const void* k, const void* v, const void* g, const float* decay,
                           const float* decay_bias, const float* bonus, const float* norm_w, void* out,
                           float* raw, const int* cu, const int* seq_slots, float* S, int num_seqs, int tokens,
                           int heads, int d, float eps, int act_type, hipStream_t stream) {
    if (num_seqs <= 0 || tokens <= 0) return RL_OK;
    if (heads < 1 || heads > 65535 || d < 1 || d > 256 || num_seqs > 65535) return RL_ERR_ARG;
    if (act_type == RL_F32)
        return launch_wkv<float>((const float*)r, (const float*)k, (const float*)v, (const float*)g, decay,
                                 decay_bias, bonus, norm_w, (float*)out, raw, cu, seq_slots, S, num_seqs, tokens,
                                 heads, d, eps, stream);
    if (act_type == RL_BF16)
        return launch_wkv<bf16_t>((const bf16_t*)r, (const bf16_t*)k, (const bf16_t*)v, (const bf16_t*)g, decay,
                                  decay_bias, bonus, norm_w, (bf16_t*)out, raw, cu, seq_slots, S, num_seqs, tokens,
                                  heads, d, eps, stream);
    return RL_ERR_ARG;
}

extern "C" int rl_causal_conv(const void* packed, int row_width, int col0, const float* w, const float* bias,
                              float* state, float* out, const int* cu, const int* seq_slots, int num_seqs,
                              int tokens, int channels, int taps, int act_type, hipStream_t stream) {
    if (tokens <= 0 || num_seqs <= 0) return RL_OK;
    if (channels < 1 || taps < 1 || taps > RL_CONV_MAX_TAPS || col0 < 0 || col0 + channels > row_width)
        return RL_ERR_ARG;
    const int cblocks = (channels + 255) / 256;
    const int single = tokens == num_seqs;  // every request brings one token
    if (cblocks > 65535) return RL_ERR_ARG;
    // single tokens: a workgroup a token, so that no token waits for another
    const int per_group = single ? 1 : recurrent::CONV_TOKENS;
    dim3 grid((tokens + per_group - 1) / per_group, cblocks), sgrid(num_seqs, cblocks);
    if (act_type == RL_F32) {
        hipLaunchKernelGGL(recurrent::causal_conv_kernel<float>, grid, dim3(256), 0, stream, (const float*)packed,
                           row_width, col0, w, bias, state, out, cu, seq_slots, num_seqs, tokens, channels, taps, single, per_group);
        if (taps > 1 && !single)
            hipLaunchKernelGGL(recurrent::conv_state_kernel<float>, sgrid, dim3(256), 0, stream,
                               (const float*)packed, row_width, col0, state, cu, seq_slots, channels, taps);
    } else if (act_type == RL_BF16) {
        hipLaunchKernelGGL(recurrent::causal_conv_kernel<bf16_t>, grid, dim3(256), 0, stream, (const bf16_t*)packed,
                           row_width, col0, w, bias, state, out, cu, seq_slots, num_seqs, tokens, channels, taps, single, per_group);
        if (taps > 1 && !single)
            hipLaunchKernelGGL(recurrent::conv_state_kernel<bf16_t>, sgrid, dim3(256), 0, stream,
                               (const bf16_t*)packed, row_width, col0, state, cu, seq_slots, channels, taps);
    } else {
        return RL_ERR_ARG;
    }
    return rl_launch_status();
}

template <typename T>
static int launch_ssm(const float* mixed, const float* dt_raw, const float* dt_bias, const float* a_log,
                      const float* skip, const T* packed, int row_width, float* out, const int* cu,
                      const int* seq_slots, float* S, int num_seqs, int tokens, int heads, int P, int N, int groups,
                      hipStream_t stream) {
    dim3 grid(num_seqs, heads, (P + recurrent::SCAN_COLS - 1) / recurrent::SCAN_COLS);
#define RL_SSM(RPL)                                                                                           \
    hipLaunchKernelGGL((recurrent::ssm_scan_kernel<T, RPL>), grid, dim3(recurrent::SCAN_THREADS), 0, stream, mixed, \
                       dt_raw, dt_bias, a_log, skip, packed, row_width, out, cu, seq_slots, S, heads, P, N, groups)
    const int rows = (N + 15) / 16;
    if (rows <= 1)
        RL_SSM(1);
    else if (rows <= 2)
        RL_SSM(2);
    else if (rows <= 4)
        RL_SSM(4);
    else if (rows <= 8)
        RL_SSM(8);
    else
        RL_SSM(16);
#undef RL_SSM
    return rl_launch_status();
}

extern "C" int rl_ssm_scan(const float* mixed, const float* dt_raw, const float* dt_bias, const float* a_log,
                           const float* skip, const void* packed, int row_width, float* out,
                           const int* cu, const int* seq_slots, float* S, int num_seqs, int tokens, int heads, int P,
                           int N, int groups, int act_type, hipStream_t stream) {
    if (num_seqs <= 0 || tokens <= 0) return RL_OK;
    if (heads < 1 || heads > 65535 || groups < 1 || heads % groups || P < 1 || P > 256 || N < 1 || N > 256 ||
        row_width < heads * P || num_seqs > 65535)
        return RL_ERR_ARG;
    if (act_type == RL_F32)
        return launch_ssm<float>(mixed, dt_raw, dt_bias, a_log, skip, (const float*)packed, row_width, out, cu,
                                 seq_slots, S, num_seqs, tokens, heads, P, N, groups, stream);
    if (act_type == RL_BF16)
        return launch_ssm<bf16_t>(mixed, dt_raw, dt_bias, a_log, skip, (const bf16_t*)packed, row_width, out,
                                  cu, seq_slots, S, num_seqs, tokens, heads, P, N, groups, stream);
    return RL_ERR_ARG;
}

extern "C" int rl_group_rmsnorm(const float* y, const float* w, void* out, int tokens, int width, int parts,
                                float eps, int act_type, hipStream_t stream) {
    if (tokens <= 0) return RL_OK;
    if (width < 1 || parts < 1 || width % parts || parts > 65535) return RL_ERR_ARG;
    dim3 grid(tokens, parts);
    if (act_type == RL_F32)
        hipLaunchKernelGGL(recurrent::group_rmsnorm_kernel<float>, grid, dim3(256), 0, stream, y, w, (float*)out,
                           width, parts, eps);
    else if (act_type == RL_BF16)
        hipLaunchKernelGGL(recurrent::group_rmsnorm_kernel<bf16_t>, grid, dim3(256), 0, stream, y, w, (bf16_t*)out,
                           width, parts, eps);
    else
        return RL_ERR_ARG;
    return rl_launch_status();
}
