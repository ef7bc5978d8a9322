// Row kernels of mixers that attend through a latent, of layer norms and of blocks whose two
// sub-layers read the same stream.
//
//   rl_add_layernorm    residual += d1 + d2 (float32, in place), then one or two layer norms
//                       (weight and bias each) of the same row: the statistics are shared
//   rl_latent_rows      from the packed row of a latent mixer's first product: the query
//                       latent RMS-normed, the key/value latent RMS-normed, the shared key part
//                       rotated, and both written into the token's place of the paged cache
//   rl_rotate_tail      the rotated part of every query head, laid behind the head's latent part
//   rl_head_product     y[t, h, :] = W_h x[t, h, :] for every head h: one small matrix a head
//                       (matrix cores for sizes in steps of 16, multiply-adds otherwise), with
//                       an optional sigmoid gate per head on the result
//
// Statistics, angles and the residual sum are float32 in both types.
#include "common.h"

namespace latent {

template <typename T>
struct alignas(sizeof(T) * 4) Vec4 {
    T v[4];
};

// --------------------------------------------------------------------------- //
// residual += d1 + d2; xhat = (x - mean) / sqrt(var + eps), var the mean of the squared
// deviations; out1 = xhat * w1 + b1, out2 = xhat * w2 + b2 (out2 may be null).  One block a
// produced row; `rows` selects which rows are produced, packed in order.  The deviations are
// taken from the mean in a second pass over the row (in registers where it fits, read again
// otherwise), not from the mean of squares.
// --------------------------------------------------------------------------- //
template <typename T, int CHUNKS>
__global__ void add_layernorm_vec_kernel(float* __restrict__ residual, const T* __restrict__ d1,
                                         const T* __restrict__ d2, const float* __restrict__ w1,
                                         const float* __restrict__ b1, T* __restrict__ out1,
                                         const float* __restrict__ w2, const float* __restrict__ b2,
                                         T* __restrict__ out2, const int* __restrict__ rows, int hidden, float eps) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int row = rows ? rows[r] : r;
    float4* res = reinterpret_cast<float4*>(residual + (size_t)row * hidden);
    const Vec4<T>* a = d1 ? reinterpret_cast<const Vec4<T>*>(d1 + (size_t)row * hidden) : nullptr;
    const Vec4<T>* b = d2 ? reinterpret_cast<const Vec4<T>*>(d2 + (size_t)row * hidden) : nullptr;
    const int nvec = hidden >> 2;
    float4 val[CHUNKS];
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int i = threadIdx.x + c * blockDim.x;
        val[c] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (i < nvec) {
            float4 v = res[i];
            if (a || b) {
                // the two sub-layers' outputs are added to each other first, then to the stream
                float4 d = make_float4(0.f, 0.f, 0.f, 0.f);
                if (a) {
                    const Vec4<T> x = a[i];
                    d = make_float4(to_float(x.v[0]), to_float(x.v[1]), to_float(x.v[2]), to_float(x.v[3]));
                }
                if (b) {
                    const Vec4<T> x = b[i];
                    d.x += to_float(x.v[0]);
                    d.y += to_float(x.v[1]);
                    d.z += to_float(x.v[2]);
                    d.w += to_float(x.v[3]);
                }
                v.x += d.x;
                v.y += d.y;
                v.z += d.z;
                v.w += d.w;
                res[i] = v;
            }
            val[c] = v;
            sum += (v.x + v.y) + (v.z + v.w);
        }
    }
    if (!out1) return;
    const float mean = block_sum(sum, scratch) / (float)hidden;
    float sq = 0.f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int i = threadIdx.x + c * blockDim.x;
        if (i < nvec) {
            val[c].x -= mean;
            val[c].y -= mean;
            val[c].z -= mean;
            val[c].w -= mean;
            sq += val[c].x * val[c].x + val[c].y * val[c].y + val[c].z * val[c].z + val[c].w * val[c].w;
        }
    }
    const float inv = 1.f / sqrtf(block_sum(sq, scratch) / (float)hidden + eps);
    const float4* w1v = reinterpret_cast<const float4*>(w1);
    const float4* b1v = reinterpret_cast<const float4*>(b1);
    const float4* w2v = reinterpret_cast<const float4*>(w2);
    const float4* b2v = reinterpret_cast<const float4*>(b2);
    Vec4<T>* o1 = reinterpret_cast<Vec4<T>*>(out1 + (size_t)r * hidden);
    Vec4<T>* o2 = out2 ? reinterpret_cast<Vec4<T>*>(out2 + (size_t)r * hidden) : nullptr;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int i = threadIdx.x + c * blockDim.x;
        if (i < nvec) {
            const float4 x = make_float4(val[c].x * inv, val[c].y * inv, val[c].z * inv, val[c].w * inv);
            {
                const float4 w = w1v[i], bb = b1v[i];
                Vec4<T> y;
                y.v[0] = from_float<T>(x.x * w.x + bb.x);
                y.v[1] = from_float<T>(x.y * w.y + bb.y);
                y.v[2] = from_float<T>(x.z * w.z + bb.z);
                y.v[3] = from_float<T>(x.w * w.w + bb.w);
                o1[i] = y;
            }
            if (o2) {
                const float4 w = w2v[i], bb = b2v[i];
                Vec4<T> y;
                y.v[0] = from_float<T>(x.x * w.x + bb.x);
                y.v[1] = from_float<T>(x.y * w.y + bb.y);
                y.v[2] = from_float<T>(x.z * w.z + bb.z);
                y.v[3] = from_float<T>(x.w * w.w + bb.w);
                o2[i] = y;
            }
        }
    }
}

// any width: element by element, the row read again for each pass
template <typename T>
__global__ void add_layernorm_kernel(float* __restrict__ residual, const T* __restrict__ d1,
                                     const T* __restrict__ d2, const float* __restrict__ w1,
                                     const float* __restrict__ b1, T* __restrict__ out1,
                                     const float* __restrict__ w2, const float* __restrict__ b2,
                                     T* __restrict__ out2, const int* __restrict__ rows, int hidden, float eps) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int row = rows ? rows[r] : r;
    float* res = residual + (size_t)row * hidden;
    const T* a = d1 ? d1 + (size_t)row * hidden : nullptr;
    const T* b = d2 ? d2 + (size_t)row * hidden : nullptr;
    float sum = 0.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float v = res[i];
        if (a || b) {
            float d = a ? to_float(a[i]) : 0.f;
            if (b) d += to_float(b[i]);
            v += d;
            res[i] = v;
        }
        sum += v;
    }
    if (!out1) return;
    const float mean = block_sum(sum, scratch) / (float)hidden;
    float sq = 0.f;
    // every thread reads back exactly the elements it wrote
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        const float dev = res[i] - mean;
        sq += dev * dev;
    }
    const float inv = 1.f / sqrtf(block_sum(sq, scratch) / (float)hidden + eps);
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        const float x = (res[i] - mean) * inv;
        out1[(size_t)r * hidden + i] = from_float<T>(x * w1[i] + b1[i]);
        if (out2) out2[(size_t)r * hidden + i] = from_float<T>(x * w2[i] + b2[i]);
    }
}

template <typename T>
static void launch_add_layernorm(float* residual, const T* d1, const T* d2, const float* w1, const float* b1,
                                 T* out1, const float* w2, const float* b2, T* out2, const int* rows,
                                 int out_rows, int hidden, float eps, hipStream_t stream) {
    dim3 grid(out_rows);
    if (hidden % 4 == 0 && hidden <= 16 * 1024) {
        const int nvec = hidden / 4;
        const int threads = ((nvec + RL_WAVE - 1) / RL_WAVE) * RL_WAVE;
        if (threads <= 1024)
            hipLaunchKernelGGL((add_layernorm_vec_kernel<T, 1>), grid, dim3(threads), 0, stream, residual, d1, d2,
                               w1, b1, out1, w2, b2, out2, rows, hidden, eps);
        else
            hipLaunchKernelGGL((add_layernorm_vec_kernel<T, 4>), grid, dim3(1024), 0, stream, residual, d1, d2,
                               w1, b1, out1, w2, b2, out2, rows, hidden, eps);
        return;
    }
    const int threads = hidden >= 2048 ? 512 : (hidden >= 512 ? 256 : 64);
    hipLaunchKernelGGL(add_layernorm_kernel<T>, grid, dim3(threads), 0, stream, residual, d1, d2, w1, b1, out1,
                       w2, b2, out2, rows, hidden, eps);
}

// --------------------------------------------------------------------------- //
// One block a token over the packed row x[t] of a latent mixer's first product:
//   columns [0, q_rank): the query latent; cq[t] = rmsnorm(.) * wq            (q_rank 0: none)
//   columns [kv_col, kv_col + r): the key/value latent c = rmsnorm(.) * wkv
//   columns [kv_col + r, kv_col + r + rd): the key part shared by all heads; its first 2 * half
//     channels rotate as pairs (2i, 2i + 1) by the token's angle, the rest pass
// and, with pages given, the token's cache row k[page, slot, :] = [c | rotated part] and the
// transposed copy of c, v[page, channel, slot].  Norm statistics float32.
// --------------------------------------------------------------------------- //
template <typename T>
__global__ __launch_bounds__(256) void latent_rows_kernel(
    const T* __restrict__ x, int row_width, int q_rank, const float* __restrict__ wq, T* __restrict__ cq,
    int kv_col, int r, int rd, const float* __restrict__ wkv, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int half, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const int* __restrict__ positions, const int* __restrict__ token_slot, const int* __restrict__ block_table,
    int table_stride, int page_size, float eps) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const T* row = x + (size_t)t * row_width;
    if (q_rank > 0) {
        float ss = 0.f;
        for (int i = threadIdx.x; i < q_rank; i += blockDim.x) {
            const float v = to_float(row[i]);
            ss += v * v;
        }
        const float f = 1.f / sqrtf(block_sum(ss, scratch) / (float)q_rank + eps);
        for (int i = threadIdx.x; i < q_rank; i += blockDim.x)
            cq[(size_t)t * q_rank + i] = from_float<T>(to_float(row[i]) * f * wq[i]);
    }
    if (!k_cache) return;
    const int pos = positions[t];
    const int page = block_table[(size_t)token_slot[t] * table_stride + pos / page_size];
    const int slot = pos % page_size;
    const T* lat = row + kv_col;
    float ss = 0.f;
    for (int i = threadIdx.x; i < r; i += blockDim.x) {
        const float v = to_float(lat[i]);
        ss += v * v;
    }
    const float f = 1.f / sqrtf(block_sum(ss, scratch) / (float)r + eps);
    T* krow = k_cache + ((size_t)page * page_size + slot) * (r + rd);
    T* vcol = v_cache + (size_t)page * r * page_size + slot;
    for (int i = threadIdx.x; i < r; i += blockDim.x) {
        const T c = from_float<T>(to_float(lat[i]) * f * wkv[i]);
        krow[i] = c;
        vcol[(size_t)i * page_size] = c;
    }
    const T* kr = lat + r;
    for (int i = threadIdx.x; i < rd / 2; i += blockDim.x) {
        const float u = to_float(kr[2 * i]), v = to_float(kr[2 * i + 1]);
        if (i < half) {
            const float c = cos_t[(size_t)pos * half + i], s = sin_t[(size_t)pos * half + i];
            krow[r + 2 * i] = from_float<T>(u * c - v * s);
            krow[r + 2 * i + 1] = from_float<T>(v * c + u * s);
        } else {
            krow[r + 2 * i] = kr[2 * i];
            krow[r + 2 * i + 1] = kr[2 * i + 1];
        }
    }
}

// --------------------------------------------------------------------------- //
// q (rows of q_row elements that begin with heads * (d + rd) channels) -> out[t, h, off .. off + rd)
// (rows of `out_width` per head): the last rd channels of every head, of which the first
// 2 * half rotate as pairs (2i, 2i + 1).
// --------------------------------------------------------------------------- //
template <typename T>
__global__ void rotate_tail_kernel(const T* __restrict__ q, T* __restrict__ out, const float* __restrict__ cos_t,
                                   const float* __restrict__ sin_t, const int* __restrict__ positions, int heads,
                                   int d, int rd, int half, int out_width, int off, int q_row, size_t total) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    const int pairs = rd / 2;
    for (; idx < total; idx += step) {
        const int i = (int)(idx % pairs);
        const size_t th = idx / pairs;  // token * heads + head
        const size_t t = th / heads;
        const int pos = positions[t];
        const T* src = q + t * q_row + (th - t * heads) * (size_t)(d + rd) + d + 2 * i;
        T* dst = out + th * (size_t)out_width + off + 2 * i;
        if (i < half) {
            const float u = to_float(src[0]), v = to_float(src[1]);
            const float c = cos_t[(size_t)pos * half + i], s = sin_t[(size_t)pos * half + i];
            dst[0] = from_float<T>(u * c - v * s);
            dst[1] = from_float<T>(v * c + u * s);
        } else {
            dst[0] = src[0];
            dst[1] = src[1];
        }
    }
}

// --------------------------------------------------------------------------- //
// y[t, h, o] = sum_i W[h, o, i] x[t, h, i]: x rows of x_row elements with head h at
// x_off + h * x_head, y likewise; W [heads, O, I] contiguous.  Optional gate: the result is
// multiplied by sigmoid(gate[t * gate_row + gate_col + h]).
// --------------------------------------------------------------------------- //
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

__device__ inline f32x4 mma(f32x4 a, f32x4 b, f32x4 acc) {
#pragma unroll
    for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j], b[j], acc, 0, 0, 0);
    return acc;
}
__device__ inline f32x4 mma(s16x4 a, s16x4 b, f32x4 acc) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, acc, 0, 0, 0);
}
template <typename T>
struct Quad;
template <>
struct Quad<float> {
    typedef f32x4 type;
};
template <>
struct Quad<bf16_t> {
    typedef s16x4 type;
};

// One wave a (16 tokens, head, 16 outputs) tile: the weights are the first operand (lane
// (o, g) holds inputs 4g .. 4g + 3 of its output row), the tokens the second (lane (t, g) the
// same inputs of its token), and a lane ends with outputs 4g .. 4g + 3 of its own token.  The sum
// over the inputs runs in ascending chunks of 16 whatever the step holds.
// CH > 0: the head has exactly CH chunks of inputs, and all of a tile's operands are read before
// the first product (a step of a few tokens is all latency here); CH 0: any number of chunks.
template <typename T, int WAVES, int CH>
__global__ __launch_bounds__(WAVES* RL_WAVE) void head_product_mfma_kernel(
    const T* __restrict__ x, const T* __restrict__ w, T* __restrict__ y, int tokens, int I, int O, int x_row,
    int x_head, int x_off, int y_row, int y_head, int y_off, const T* __restrict__ gate, int gate_row,
    int gate_col) {
    typedef typename Quad<T>::type quad;
    const int lane = threadIdx.x & (RL_WAVE - 1);
    const int wave = threadIdx.x / RL_WAVE;
    const int r16 = lane & 15, g = lane >> 4;
    const int h = blockIdx.y;
    const int o0 = 16 * (blockIdx.z * WAVES + wave);
    if (o0 >= O) return;
    const int t0 = 16 * blockIdx.x;
    const int t = min(t0 + r16, tokens - 1);
    const T* xr = x + (size_t)t * x_row + x_off + (size_t)h * x_head + 4 * g;
    const T* wr = w + ((size_t)h * O + o0 + r16) * I + 4 * g;
    f32x4 acc = (f32x4){0.f, 0.f, 0.f, 0.f};
    const int chunks = I / 16;
    int c = 0;
    if (CH > 0) {
        quad a[CH > 0 ? CH : 1], b[CH > 0 ? CH : 1];
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            a[j] = *reinterpret_cast<const quad*>(wr + 16 * j);
            b[j] = *reinterpret_cast<const quad*>(xr + 16 * j);
        }
#pragma unroll
        for (int j = 0; j < CH; ++j) acc = mma(a[j], b[j], acc);
        c = chunks;
    }
    // four chunks' operands are read before their products: the reads are in flight together
    for (; c + 4 <= chunks; c += 4) {
        quad a[4], b[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            a[j] = *reinterpret_cast<const quad*>(wr + 16 * (c + j));
            b[j] = *reinterpret_cast<const quad*>(xr + 16 * (c + j));
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = mma(a[j], b[j], acc);
    }
    for (; c < chunks; ++c) {
        const quad a = *reinterpret_cast<const quad*>(wr + 16 * c);
        const quad b = *reinterpret_cast<const quad*>(xr + 16 * c);
        acc = mma(a, b, acc);
    }
    if (t0 + r16 >= tokens) return;
    float f = 1.f;
    if (gate) f = 1.f / (1.f + expf(-to_float(gate[(size_t)t * gate_row + gate_col + h])));
    T* yr = y + (size_t)t * y_row + y_off + (size_t)h * y_head + o0 + 4 * g;
    Vec4<T> out;
#pragma unroll
    for (int i = 0; i < 4; ++i) out.v[i] = from_float<T>(acc[i] * f);
    *reinterpret_cast<Vec4<T>*>(yr) = out;
}

// Blocks of 16 tokens a wave keeps in registers in a step of many tokens: as many as 64 registers
// a lane hold of CH chunks of inputs.
template <typename T, int CH>
constexpr int head_rows_blocks() {
    constexpr int regs = CH * (int)sizeof(typename Quad<T>::type) / 4;
    return regs * 4 <= 64 ? 4 : (regs * 2 <= 64 ? 2 : 1);
}

// Steps of many tokens: one wave a (TB blocks of 16 tokens, head) pair.  The wave keeps its tokens'
// inputs in registers (CH chunks of 16 a block) and walks the head's output tiles: a token's inputs
// are read once, and every read of the head's matrix (16 rows of a few bytes each, which the load
// path takes one cache line after the other) serves TB blocks of tokens.  Every output's sum runs
// over the same chunks in the same order as in the kernel above: the same bits.  EXACT: the head
// has exactly CH chunks of inputs and no read hangs on a comparison.
template <typename T, int WAVES, int CH, bool EXACT>
__global__ __launch_bounds__(WAVES* RL_WAVE) void head_product_rows_kernel(
    const T* __restrict__ x, const T* __restrict__ w, T* __restrict__ y, int tokens, int I, int O, int x_row,
    int x_head, int x_off, int y_row, int y_head, int y_off, const T* __restrict__ gate, int gate_row,
    int gate_col) {
    typedef typename Quad<T>::type quad;
    constexpr int TB = head_rows_blocks<T, CH>();
    const int lane = threadIdx.x & (RL_WAVE - 1);
    const int wave = threadIdx.x / RL_WAVE;
    const int r16 = lane & 15, g = lane >> 4;
    const int h = blockIdx.y;
    const int t0 = 16 * TB * (blockIdx.x * WAVES + wave);
    if (t0 >= tokens) return;
    const int chunks = I / 16;
    quad xs[TB][CH];
    float f[TB];
    int t[TB];
#pragma unroll
    for (int b = 0; b < TB; ++b) {
        t[b] = min(t0 + 16 * b + r16, tokens - 1);
        const T* xr = x + (size_t)t[b] * x_row + x_off + (size_t)h * x_head + 4 * g;
#pragma unroll
        for (int c = 0; c < CH; ++c)
            if (EXACT || c < chunks) xs[b][c] = *reinterpret_cast<const quad*>(xr + 16 * c);
        f[b] = 1.f;
        if (gate) f[b] = 1.f / (1.f + expf(-to_float(gate[(size_t)t[b] * gate_row + gate_col + h])));
    }
    // blockIdx.z deals the output tiles to gridDim.z workgroups: more waves in flight where a head
    // has many outputs
    const int per = ((O / 16 + gridDim.z - 1) / gridDim.z) * 16;
    const int o_end = min(O, (int)(blockIdx.z + 1) * per);
    for (int o0 = blockIdx.z * per; o0 < o_end; o0 += 16) {
        const T* wr = w + ((size_t)h * O + o0 + r16) * I + 4 * g;
        f32x4 acc[TB];
#pragma unroll
        for (int b = 0; b < TB; ++b) acc[b] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < CH; ++c)
            if (EXACT || c < chunks) {
                const quad a = *reinterpret_cast<const quad*>(wr + 16 * c);
#pragma unroll
                for (int b = 0; b < TB; ++b) acc[b] = mma(a, xs[b][c], acc[b]);
            }
#pragma unroll
        for (int b = 0; b < TB; ++b)
            if (t0 + 16 * b + r16 < tokens) {
                Vec4<T> out;
#pragma unroll
                for (int i = 0; i < 4; ++i) out.v[i] = from_float<T>(acc[b][i] * f[b]);
                *reinterpret_cast<Vec4<T>*>(y + (size_t)t[b] * y_row + y_off + (size_t)h * y_head + 4 * g + o0) = out;
            }
    }
}

// any sizes: one thread an output element
template <typename T>
__global__ void head_product_kernel(const T* __restrict__ x, const T* __restrict__ w, T* __restrict__ y,
                                    int heads, int I, int O, int x_row, int x_head, int x_off, int y_row,
                                    int y_head, int y_off, const T* __restrict__ gate, int gate_row, int gate_col,
                                    size_t total) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (; idx < total; idx += step) {
        const int o = (int)(idx % O);
        const size_t th = idx / O;
        const int h = (int)(th % heads);
        const size_t t = th / heads;
        const T* xr = x + t * x_row + x_off + (size_t)h * x_head;
        const T* wr = w + ((size_t)h * O + o) * I;
        float acc = 0.f;
        for (int i = 0; i < I; ++i) acc = fmaf(to_float(wr[i]), to_float(xr[i]), acc);
        if (gate) acc /= 1.f + expf(-to_float(gate[t * gate_row + gate_col + h]));
        y[t * y_row + y_off + (size_t)h * y_head + o] = from_float<T>(acc);
    }
}

}  // namespace latent

extern "C" int rl_add_layernorm(float* residual, const void* d1, const void* d2, const float* w1, const float* b1,
                                void* out1, const float* w2, const float* b2, void* out2, const int* rows,
                                int out_rows, int hidden, float eps, int act_type, hipStream_t stream) {
    if (out_rows <= 0 || hidden <= 0) return RL_OK;
    if (out1 && (!w1 || !b1)) return RL_ERR_ARG;
    if (out2 && (!out1 || !w2 || !b2)) return RL_ERR_ARG;
    if (act_type == RL_F32)
        latent::launch_add_layernorm<float>(residual, (const float*)d1, (const float*)d2, w1, b1, (float*)out1, w2, b2,
                                            (float*)out2, rows, out_rows, hidden, eps, stream);
    else if (act_type == RL_BF16)
        latent::launch_add_layernorm<bf16_t>(residual, (const bf16_t*)d1, (const bf16_t*)d2, w1, b1, (bf16_t*)out1,
                                             w2, b2, (bf16_t*)out2, rows, out_rows, hidden, eps, stream);
    else
        return RL_ERR_ARG;
    return rl_launch_status();
}

extern "C" int rl_latent_rows(const void* x, int row_width, int tokens, int q_rank, const float* wq, void* cq,
                              int kv_col, int r, int rd, const float* wkv, const float* cos_t, const float* sin_t,
                              int half, void* k_cache, void* v_cache, const int* positions, const int* token_slot,
                              const int* block_table, int table_stride, int page_size, float eps, int act_type,
                              hipStream_t stream) {
    if (tokens <= 0) return RL_OK;
    if (q_rank < 0 || (q_rank > 0 && (!wq || !cq)) || q_rank > row_width) return RL_ERR_ARG;
    if (k_cache) {
        if (!v_cache || !wkv || r < 1 || rd < 0 || rd % 2 || half < 0 || 2 * half > rd || kv_col < 0 ||
            kv_col + r + rd > row_width || page_size < 1 || (half > 0 && (!cos_t || !sin_t)))
            return RL_ERR_ARG;
    } else if (q_rank == 0) {
        return RL_OK;
    }
    dim3 grid(tokens), block(256);
    if (act_type == RL_F32)
        hipLaunchKernelGGL(latent::latent_rows_kernel<float>, grid, block, 0, stream, (const float*)x, row_width,
                           q_rank, wq, (float*)cq, kv_col, r, rd, wkv, cos_t, sin_t, half, (float*)k_cache,
                           (float*)v_cache, positions, token_slot, block_table, table_stride, page_size, eps);
    else if (act_type == RL_BF16)
        hipLaunchKernelGGL(latent::latent_rows_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)x, row_width,
                           q_rank, wq, (bf16_t*)cq, kv_col, r, rd, wkv, cos_t, sin_t, half, (bf16_t*)k_cache,
                           (bf16_t*)v_cache, positions, token_slot, block_table, table_stride, page_size, eps);
    else
        return RL_ERR_ARG;
    return rl_launch_status();
}

extern "C" int rl_rotate_tail(const void* q, void* out, const float* cos_t, const float* sin_t,
                              const int* positions, int tokens, int heads, int d, int rd, int half, int out_width,
                              int off, int q_row, int act_type, hipStream_t stream) {
    if (tokens <= 0 || heads <= 0 || rd <= 0) return RL_OK;
    if (rd % 2 || half < 0 || 2 * half > rd || d < 0 || off < 0 || off + rd > out_width ||
        q_row < heads * (d + rd) ||
        (half > 0 && (!cos_t || !sin_t)))
        return RL_ERR_ARG;
    const size_t total = (size_t)tokens * heads * (rd / 2);
    size_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    dim3 grid((unsigned)blocks), block(256);
    if (act_type == RL_F32)
        hipLaunchKernelGGL(latent::rotate_tail_kernel<float>, grid, block, 0, stream, (const float*)q, (float*)out,
                           cos_t, sin_t, positions, heads, d, rd, half, out_width, off, q_row, total);
    else if (act_type == RL_BF16)
        hipLaunchKernelGGL(latent::rotate_tail_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)q,
                           (bf16_t*)out, cos_t, sin_t, positions, heads, d, rd, half, out_width, off, q_row, total);
    else
        return RL_ERR_ARG;
    return rl_launch_status();
}

extern "C" int rl_head_product(const void* x, const void* w, void* y, int tokens, int heads, int I, int O,
                               int x_row, int x_head, int x_off, int y_row, int y_head, int y_off,
                               const void* gate, int gate_row, int gate_col, int act_type, hipStream_t stream) {
    if (tokens <= 0 || heads <= 0 || O <= 0) return RL_OK;
    if (I < 1 || heads > 65535 || x_off < 0 || y_off < 0) return RL_ERR_ARG;
    if (act_type != RL_F32 && act_type != RL_BF16) return RL_ERR_ARG;
    // the matrix cores read four consecutive elements a lane: every offset a multiple of four
    const bool tiles = I % 16 == 0 && O % 16 == 0 && x_row % 4 == 0 && x_head % 4 == 0 && x_off % 4 == 0 &&
                       y_row % 4 == 0 && y_head % 4 == 0 && y_off % 4 == 0;
    // from this many tokens on a wave keeps 16 tokens' inputs and walks the outputs: below it the
    // launch of a tile a wave has more waves than the chip has units to give them
    if (tiles && tokens >= 256 && I <= 512) {
        constexpr int WAVES = 4;
        const int otiles = O / 16;
        dim3 grid(1, heads, otiles >= 16 ? 4 : (otiles >= 4 ? 2 : 1));
        dim3 block(WAVES * RL_WAVE);
#define RL_HEAD_ROWS(TYPE, CH, EXACT)                                                                              \
    do {                                                                                                             \
        grid.x = (tokens + 16 * WAVES * latent::head_rows_blocks<TYPE, CH>() - 1) /                                    \
                 (16 * WAVES * latent::head_rows_blocks<TYPE, CH>());                                                  \
        hipLaunchKernelGGL((latent::head_product_rows_kernel<TYPE, WAVES, CH, EXACT>), grid, block, 0, stream,          \
                           (const TYPE*)x, (const TYPE*)w, (TYPE*)y, tokens, I, O, x_row, x_head, x_off, y_row, y_head, \
                           y_off, (const TYPE*)gate, gate_row, gate_col);                                               \
    } while (0)
#define RL_HEAD_ROWS_OF(TYPE)                       \
    switch (I / 16) {                               \
        case 1: RL_HEAD_ROWS(TYPE, 1, true); break;   \
        case 2: RL_HEAD_ROWS(TYPE, 2, true); break;   \
        case 4: RL_HEAD_ROWS(TYPE, 4, true); break;   \
        case 8: RL_HEAD_ROWS(TYPE, 8, true); break;   \
        case 16: RL_HEAD_ROWS(TYPE, 16, true); break; \
        case 32: RL_HEAD_ROWS(TYPE, 32, true); break; \
        default:                                    \
            if (I <= 128) RL_HEAD_ROWS(TYPE, 8, false);       \
            else if (I <= 256) RL_HEAD_ROWS(TYPE, 16, false); \
            else RL_HEAD_ROWS(TYPE, 32, false);               \
    }
        if (act_type == RL_F32) {
            RL_HEAD_ROWS_OF(float)
        } else {
            RL_HEAD_ROWS_OF(bf16_t)
        }
#undef RL_HEAD_ROWS_OF
#undef RL_HEAD_ROWS
        return rl_launch_status();
    }
    if (tiles) {
        constexpr int WAVES = 4;
        const int otiles = O / 16;
        dim3 grid((tokens + 15) / 16, heads, (otiles + WAVES - 1) / WAVES), block(WAVES * RL_WAVE);
        if (grid.z > 65535) return RL_ERR_ARG;
#define RL_HEAD_TILE(TYPE, CH)                                                                                    \
    hipLaunchKernelGGL((latent::head_product_mfma_kernel<TYPE, WAVES, CH>), grid, block, 0, stream, (const TYPE*)x, \
                       (const TYPE*)w, (TYPE*)y, tokens, I, O, x_row, x_head, x_off, y_row, y_head, y_off,          \
                       (const TYPE*)gate, gate_row, gate_col)
#define RL_HEAD_TILE_OF(TYPE)                  \
    switch (I / 16) {                          \
        case 1: RL_HEAD_TILE(TYPE, 1); break;   \
        case 2: RL_HEAD_TILE(TYPE, 2); break;   \
        case 4: RL_HEAD_TILE(TYPE, 4); break;   \
        case 8: RL_HEAD_TILE(TYPE, 8); break;   \
        case 16: RL_HEAD_TILE(TYPE, 16); break; \
        default: RL_HEAD_TILE(TYPE, 0);         \
    }
        if (act_type == RL_F32) {
            RL_HEAD_TILE_OF(float)
        } else {
            RL_HEAD_TILE_OF(bf16_t)
        }
#undef RL_HEAD_TILE_OF
#undef RL_HEAD_TILE
        return rl_launch_status();
    }
    const size_t total = (size_t)tokens * heads * O;
    size_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    dim3 grid((unsigned)blocks), block(256);
    if (act_type == RL_F32)
        hipLaunchKernelGGL(latent::head_product_kernel<float>, grid, block, 0, stream, (const float*)x,
                           (const float*)w, (float*)y, heads, I, O, x_row, x_head, x_off, y_row, y_head, y_off,
                           (const float*)gate, gate_row, gate_col, total);
    else
        hipLaunchKernelGGL(latent::head_product_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)x,
                           (const bf16_t*)w, (bf16_t*)y, heads, I, O, x_row, x_head, x_off, y_row, y_head, y_off,
                           (const bf16_t*)gate, gate_row, gate_col, total);
    return rl_launch_status();
}
