// Recurrent mixers with a fixed-size state per request: the token-shift mixes and the per-head
// scan of an RWKV-style time mixing, and the causal convolution, the scan and the grouped norm of a
// state-space mixer.  Everything between the projections is float32: mixes of the decay branch,
// decays, step sizes, states, sums, norms; the element type T only says how the projections'
// results are read and the mixers' outputs written.
//
// A step is a flat batch of requests: request s brings the tokens cu[s] .. cu[s + 1] - 1 and keeps
// its state in row seq_slots[s] of the state tensors.  Every scan walks a request's tokens in
// order with the state in registers, one workgroup per (request, head), so a token's sums are
// formed in one order whatever else the step holds and however the request's tokens were cut into
// steps: in float32 the results are equal bit for bit.
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
// The state row is replaced by the request's last row in a second launch, after every read.
// --------------------------------------------------------------------------- //
template <typename T>
__global__ __launch_bounds__(256) void token_shift_kernel(const T* __restrict__ x, const float* __restrict__ mu,
                                                          const float* __restrict__ state, T* __restrict__ mixes,
                                                          float* __restrict__ mix_w, const int* __restrict__ cu,
                                                          const int* __restrict__ seq_slots, int num_seqs,
                                                          int tokens, int width) {
    const int t = blockIdx.x;
    const int s = request_of(cu, num_seqs, t);
    const bool first = t == cu[s];
    const float* prev_state = state + (size_t)seq_slots[s] * width;
    const T* row = x + (size_t)t * width;
    const T* before = x + (size_t)(first ? t : t - 1) * width;
    const size_t plane = (size_t)tokens * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float h = to_float(row[i]);
        const float p = first ? prev_state[i] : to_float(before[i]);
        const float d = p - h;
#pragma unroll
        for (int b = 0; b < 4; ++b)
            mixes[b * plane + (size_t)t * width + i] = from_float<T>(h + d * mu[(size_t)b * width + i]);
        mix_w[(size_t)t * width + i] = h + d * mu[(size_t)4 * width + i];
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
// The time-mixing scan.  Per head, state S[key channel i][value channel j]; thread j keeps column
// j in registers.  For a token with r, k, v (d each), decay w_i = exp(-exp(pre_i + bias_i)) and
// the bonus u_i:
//   o_j = sum_i r_i (S_ij + u_i k_i v_j)        S_ij <- w_i S_ij + k_i v_j
// then o is divided by its root mean square over the head, multiplied by the norm's weight and by
// silu(g).  The next token's operands travel while this one is computed.
// --------------------------------------------------------------------------- //
template <typename T, int DMAX>
__global__ __launch_bounds__(DMAX < 64 ? 64 : DMAX) void wkv_scan_kernel(
    const T* __restrict__ r, const T* __restrict__ k, const T* __restrict__ v, const T* __restrict__ g,
    const float* __restrict__ decay_pre, const float* __restrict__ decay_bias, const float* __restrict__ bonus,
    const float* __restrict__ norm_w, T* __restrict__ out, const int* __restrict__ cu,
    const int* __restrict__ seq_slots, float* __restrict__ S, int heads, int d, float eps) {
    const int s = blockIdx.x, h = blockIdx.y, j = threadIdx.x;
    const int t0 = cu[s], t1 = cu[s + 1];
    const int inner = heads * d;
    const bool live = j < d;
    const int col = h * d + (live ? j : 0);
    __shared__ float sr[DMAX], sk[DMAX], sw[DMAX], su[DMAX];
    __shared__ float scratch[16];
    float* Sp = S + ((size_t)seq_slots[s] * heads + h) * d * d;
    float state[DMAX];
#pragma unroll
    for (int i = 0; i < DMAX; ++i) state[i] = (live && i < d) ? Sp[(size_t)i * d + j] : 0.f;
    const float bias = decay_bias[col], nw = norm_w[col];
    if (live) su[j] = bonus[col];
    float nr = 0.f, nk = 0.f, nv = 0.f, ng = 0.f, np = 0.f;
    if (t0 < t1) {
        const size_t at = (size_t)t0 * inner + col;
        nr = to_float(r[at]); nk = to_float(k[at]); nv = to_float(v[at]); ng = to_float(g[at]); np = decay_pre[at];
    }
    for (int t = t0; t < t1; ++t) {
        __syncthreads();  // the token before has been read by every thread
        if (live) {
            sr[j] = nr;
            sk[j] = nk;
            sw[j] = expf(-expf(np + bias));
        }
        const float vj = live ? nv : 0.f, gj = ng;
        __syncthreads();
        if (t + 1 < t1) {
            const size_t at = (size_t)(t + 1) * inner + col;
            nr = to_float(r[at]); nk = to_float(k[at]); nv = to_float(v[at]); ng = to_float(g[at]); np = decay_pre[at];
        }
        float o = 0.f;
#pragma unroll
        for (int i = 0; i < DMAX; ++i) {
            if (i < d) {
                const float kv = sk[i] * vj;
                o += sr[i] * (state[i] + su[i] * kv);
                state[i] = sw[i] * state[i] + kv;
            }
        }
        const float ss = block_sum(live ? o * o : 0.f, scratch);
        const float rr = rsqrtf(ss / (float)d + eps);
        if (live) out[(size_t)t * inner + col] = from_float<T>(o * rr * nw * silu(gj));
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < DMAX; ++i)
            if (i < d) Sp[(size_t)i * d + j] = state[i];
    }
}

// --------------------------------------------------------------------------- //
// Causal convolution per channel over the columns [col0, col0 + channels) of the packed rows, with
// bias and silu: y_t = silu(b + sum_tap w[c][tap] in(t - (taps - 1) + tap)), where inputs before
// the request's first token of the step come from its state rows (the last taps - 1 inputs it has
// seen, oldest first; zeros when the request begins).  A second launch then shifts the state.
// --------------------------------------------------------------------------- //
#define RL_CONV_MAX_TAPS 8

template <typename T>
__global__ __launch_bounds__(256) void causal_conv_kernel(const T* __restrict__ packed, int row_width, int col0,
                                                          const float* __restrict__ w, const float* __restrict__ bias,
                                                          const float* __restrict__ state, float* __restrict__ out,
                                                          const int* __restrict__ cu,
                                                          const int* __restrict__ seq_slots, int num_seqs,
                                                          int channels, int taps) {
    const int t = blockIdx.x;
    const int s = request_of(cu, num_seqs, t);
    const int offset = t - cu[s];  // tokens of the request's portion before this one
    const int held = taps - 1;
    const float* st = state + (size_t)seq_slots[s] * max(held, 1) * channels;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < channels; c += gridDim.y * blockDim.x) {
        float acc = bias[c];
        for (int tap = 0; tap < taps; ++tap) {
            const int rel = offset - held + tap;  // offset in the portion of the input this tap meets
            const float in = rel >= 0 ? to_float(packed[(size_t)(t - offset + rel) * row_width + col0 + c])
                                      : st[(size_t)(held + rel) * channels + c];
            acc = fmaf(w[(size_t)c * taps + tap], in, acc);
        }
        out[(size_t)t * channels + c] = silu(acc);
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
// behind convolution and silu); per head, state S[n][p], thread p keeps column p in registers:
//   dt = softplus(dt_raw + dt_bias)     a = exp(-exp(A_log) dt)
//   S_np <- a S_np + dt B_n x_p          y_p = sum_n S_np C_n + D x_p
// and y_p silu(z_p) is written (z: the first heads * P columns of the packed rows).
// --------------------------------------------------------------------------- //
template <typename T, int NMAX>
__global__ __launch_bounds__(256) void ssm_scan_kernel(
    const float* __restrict__ mixed, const float* __restrict__ dt_raw, const float* __restrict__ dt_bias,
    const float* __restrict__ a_log, const float* __restrict__ skip, const T* __restrict__ packed, int row_width,
    float* __restrict__ out, const int* __restrict__ cu, const int* __restrict__ seq_slots,
    float* __restrict__ S, int heads, int P, int N, int groups) {
    const int s = blockIdx.x, h = blockIdx.y, p = threadIdx.x;
    const int t0 = cu[s], t1 = cu[s + 1];
    const int inner = heads * P;
    const int channels = inner + 2 * groups * N;
    const int grp = h / (heads / groups);
    const bool live = p < P;
    const bool feeds = p < N;  // this thread also carries B_n and C_n of n = p into LDS
    __shared__ float sB[NMAX], sC[NMAX];
    float* Sp = S + ((size_t)seq_slots[s] * heads + h) * N * P;
    float state[NMAX];
#pragma unroll
    for (int n = 0; n < NMAX; ++n) state[n] = (live && n < N) ? Sp[(size_t)n * P + p] : 0.f;
    const float bias = dt_bias[h], rate = expf(a_log[h]), D = skip[h];
    const int xcol = h * P + (live ? p : 0);
    const int bcol = inner + grp * N + (feeds ? p : 0);
    const int ccol = bcol + groups * N;
    float nx = 0.f, nb = 0.f, nc = 0.f, nz = 0.f, nd = 0.f;
    if (t0 < t1) {
        const float* row = mixed + (size_t)t0 * channels;
        nx = row[xcol]; nb = row[bcol]; nc = row[ccol];
        nz = to_float(packed[(size_t)t0 * row_width + xcol]);
        nd = dt_raw[(size_t)t0 * heads + h];
    }
    for (int t = t0; t < t1; ++t) {
        __syncthreads();  // the token before has been read by every thread
        if (feeds) {
            sB[p] = nb;
            sC[p] = nc;
        }
        const float x = live ? nx : 0.f, z = nz;
        const float pre = nd + bias;
        const float dt = pre > 20.f ? pre : log1pf(expf(pre));
        const float a = expf(-rate * dt);
        __syncthreads();
        if (t + 1 < t1) {
            const float* row = mixed + (size_t)(t + 1) * channels;
            nx = row[xcol]; nb = row[bcol]; nc = row[ccol];
            nz = to_float(packed[(size_t)(t + 1) * row_width + xcol]);
            nd = dt_raw[(size_t)(t + 1) * heads + h];
        }
        const float dx = dt * x;
        float y = 0.f;
#pragma unroll
        for (int n = 0; n < NMAX; ++n) {
            if (n < N) {
                state[n] = a * state[n] + sB[n] * dx;
                y += state[n] * sC[n];
            }
        }
        y += D * x;
        if (live) out[(size_t)t * inner + xcol] = y * silu(z);
    }
    if (live) {
#pragma unroll
        for (int n = 0; n < NMAX; ++n)
            if (n < N) Sp[(size_t)n * P + p] = state[n];
    }
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
    if (act_type == RL_F32) {
        hipLaunchKernelGGL(recurrent::token_shift_kernel<float>, dim3(tokens), dim3(256), 0, stream, (const float*)x,
                           mu, state, (float*)mixes, mix_w, cu, seq_slots, num_seqs, tokens, width);
        hipLaunchKernelGGL(recurrent::shift_state_kernel<float>, dim3(num_seqs), dim3(256), 0, stream,
                           (const float*)x, state, cu, seq_slots, width);
    } else if (act_type == RL_BF16) {
        hipLaunchKernelGGL(recurrent::token_shift_kernel<bf16_t>, dim3(tokens), dim3(256), 0, stream,
                           (const bf16_t*)x, mu, state, (bf16_t*)mixes, mix_w, cu, seq_slots, num_seqs, tokens,
                           width);
        hipLaunchKernelGGL(recurrent::shift_state_kernel<bf16_t>, dim3(num_seqs), dim3(256), 0, stream,
                           (const bf16_t*)x, state, cu, seq_slots, width);
    } else {
        return RL_ERR_ARG;
    }
    return rl_launch_status();
}

template <typename T>
static int launch_wkv(const T* r, const T* k, const T* v, const T* g, const float* decay_pre,
                      const float* decay_bias, const float* bonus, const float* norm_w, T* out, const int* cu,
                      const int* seq_slots, float* S, int num_seqs, int heads, int d, float eps,
                      hipStream_t stream) {
    dim3 grid(num_seqs, heads);
#define RL_WKV(DMAX)                                                                                            \
    hipLaunchKernelGGL((recurrent::wkv_scan_kernel<T, DMAX>), grid, dim3(DMAX < 64 ? 64 : DMAX), 0, stream, r, k, v, \
                       g, decay_pre, decay_bias, bonus, norm_w, out, cu, seq_slots, S, heads, d, eps)
    if (d <= 32)
        RL_WKV(32);
    else if (d <= 64)
        RL_WKV(64);
    else if (d <= 128)
        RL_WKV(128);
    else
        RL_WKV(256);
#undef RL_WKV
    return rl_launch_status();
}

extern "C" int rl_wkv_scan(const void* r, const void* k, const void* v, const void* g, const float* decay_pre,
                           const float* decay_bias, const float* bonus, const float* norm_w, void* out,
                           const int* cu, const int* seq_slots, float* S, int num_seqs, int heads, int d,
                           float eps, int act_type, hipStream_t stream) {
    if (num_seqs <= 0) return RL_OK;
    if (heads < 1 || heads > 65535 || d < 1 || d > 256) return RL_ERR_ARG;
    if (act_type == RL_F32)
        return launch_wkv<float>((const float*)r, (const float*)k, (const float*)v, (const float*)g, decay_pre,
                                 decay_bias, bonus, norm_w, (float*)out, cu, seq_slots, S, num_seqs, heads, d, eps,
                                 stream);
    if (act_type == RL_BF16)
        return launch_wkv<bf16_t>((const bf16_t*)r, (const bf16_t*)k, (const bf16_t*)v, (const bf16_t*)g, decay_pre,
                                  decay_bias, bonus, norm_w, (bf16_t*)out, cu, seq_slots, S, num_seqs, heads, d,
                                  eps, stream);
    return RL_ERR_ARG;
}

extern "C" int rl_causal_conv(const void* packed, int row_width, int col0, const float* w, const float* bias,
                              float* state, float* out, const int* cu, const int* seq_slots, int num_seqs,
                              int tokens, int channels, int taps, int act_type, hipStream_t stream) {
    if (tokens <= 0 || num_seqs <= 0) return RL_OK;
    if (channels < 1 || taps < 1 || taps > RL_CONV_MAX_TAPS || col0 < 0 || col0 + channels > row_width)
        return RL_ERR_ARG;
    const int cblocks = (channels + 255) / 256;
    dim3 grid(tokens, cblocks > 64 ? 64 : cblocks), sgrid(num_seqs, cblocks);
    if (act_type == RL_F32) {
        hipLaunchKernelGGL(recurrent::causal_conv_kernel<float>, grid, dim3(256), 0, stream, (const float*)packed,
                           row_width, col0, w, bias, state, out, cu, seq_slots, num_seqs, channels, taps);
        if (taps > 1)
            hipLaunchKernelGGL(recurrent::conv_state_kernel<float>, sgrid, dim3(256), 0, stream,
                               (const float*)packed, row_width, col0, state, cu, seq_slots, channels, taps);
    } else if (act_type == RL_BF16) {
        hipLaunchKernelGGL(recurrent::causal_conv_kernel<bf16_t>, grid, dim3(256), 0, stream, (const bf16_t*)packed,
                           row_width, col0, w, bias, state, out, cu, seq_slots, num_seqs, channels, taps);
        if (taps > 1)
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
                      const int* seq_slots, float* S, int num_seqs, int heads, int P, int N, int groups,
                      hipStream_t stream) {
    dim3 grid(num_seqs, heads);
    const int need = P > N ? P : N;
    dim3 block(((need + 63) / 64) * 64);
#define RL_SSM(NMAX)                                                                                             \
    hipLaunchKernelGGL((recurrent::ssm_scan_kernel<T, NMAX>), grid, block, 0, stream, mixed, dt_raw, dt_bias, a_log, \
                       skip, packed, row_width, out, cu, seq_slots, S, heads, P, N, groups)
    if (N <= 16)
        RL_SSM(16);
    else if (N <= 32)
        RL_SSM(32);
    else if (N <= 64)
        RL_SSM(64);
    else if (N <= 128)
        RL_SSM(128);
    else
        RL_SSM(256);
#undef RL_SSM
    return rl_launch_status();
}

extern "C" int rl_ssm_scan(const float* mixed, const float* dt_raw, const float* dt_bias, const float* a_log,
                           const float* skip, const void* packed, int row_width, float* out, const int* cu,
                           const int* seq_slots, float* S, int num_seqs, int heads, int P, int N, int groups,
                           int act_type, hipStream_t stream) {
    if (num_seqs <= 0) return RL_OK;
    if (heads < 1 || heads > 65535 || groups < 1 || heads % groups || P < 1 || P > 256 || N < 1 || N > 256 ||
        row_width < heads * P)
        return RL_ERR_ARG;
    if (act_type == RL_F32)
        return launch_ssm<float>(mixed, dt_raw, dt_bias, a_log, skip, (const float*)packed, row_width, out, cu,
                                 seq_slots, S, num_seqs, heads, P, N, groups, stream);
    if (act_type == RL_BF16)
        return launch_ssm<bf16_t>(mixed, dt_raw, dt_bias, a_log, skip, (const bf16_t*)packed, row_width, out, cu,
                                  seq_slots, S, num_seqs, heads, P, N, groups, stream);
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
