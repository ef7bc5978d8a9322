// Paged causal attention over tiles of 16 rows for mixers that the other attention kernels do
// not take: value heads of a size of their own, a sliding window that keeps a request's first
// positions visible, and a softmax with one more term in its denominator.  Compiled for one
// pair of head sizes RL_HEAD_DIM (queries and keys) and RL_VALUE_DIM (values), multiples of 16,
// in float32 (v_mfma_f32_16x16x4_f32: true 32-bit) and in bfloat16 (v_mfma_f32_16x16x16_bf16,
// float32 accumulation, scores and softmax state in float32, the weights rounded to bfloat16
// for the product with the values).
//
// One workgroup of AW waves per (tile of 16 rows, kv head).  Rows are (token, query head of
// the kv group) pairs of ONE request, so grouped heads and neighbouring tokens share every key
// that is read; a single token's tile holds the heads of its group.  The key tiles are dealt to
// the waves by their absolute index (tile i goes to wave i % AW), each wave keeps a softmax
// state of its own, and the states are folded in the order of the waves.  The transposed
// products are computed,
//   S^T[keys, rows] = K[keys, d] Q^T[d, rows],   O^T[dv, rows] += V^T[dv, keys] P^T[keys, rows],
// which leaves a lane with the scores of keys 4g .. 4g + 3 of its own row: exactly its operand
// of the second product, whose other operand is one read of the transposed value cache.
//
// What a row sees: key j of its request with j <= p (its position) and, with a window w > 0,
// p - j < w or j < keep_first.  The tiles walked are those of [0, keep_first) and those from
// the window of the tile's first row up to its last row's position.  With `sink` the softmax's
// denominator is 1 + sum_j exp(s_j): a key of score 0 that carries no value.
//
// Two options change a score s = (q . k) scale before the softmax: with cap > 0 it becomes
// cap * tanh(s / cap), and with `slopes` (one number a query head) slope_h * (p - j) is taken off
// it afterwards.  The sink's term has neither.
//
// A row's result does not depend on the tile it falls in, on the other rows there, or on how a
// prompt was cut into steps: keys are taken in tiles of 16 at absolute positions 0, 16, ..,
// each wave takes its tiles in ascending order; within a tile the order of every sum is fixed
// by the key's position; a tile that holds no visible key of a row leaves that row's state as
// it is, exactly (factor 1, terms 0), and so does a wave without visible keys in the fold.
// Masked keys contribute exactly zero; pages between the kept positions and the window may have
// been given back, so what is read there is never multiplied into a sum.
#include "common.h"

#ifndef RL_HEAD_DIM
#error "compile with -DRL_HEAD_DIM=<size of a query or key head>"
#endif
#ifndef RL_VALUE_DIM
#error "compile with -DRL_VALUE_DIM=<size of a value head>"
#endif

namespace tileattn {

constexpr int D = RL_HEAD_DIM;
constexpr int DV = RL_VALUE_DIM;
constexpr int DB = D / 16;   // 16-channel chunks of the first product
constexpr int VB = DV / 16;  // 16-channel blocks of the output
// blocks of 16 rows a wave multiplies with every key tile it reads, in a bfloat16 step of
// portions: as many as the registers hold beside two tiles of operands (two up to 320 + 256
// channels, where they fill every register of a lane without parking any in scratch memory)
constexpr int PORTION_BLOCKS = (D + DV <= 192) ? 4 : ((D + DV <= 576) ? 2 : 1);
constexpr int MAX_STAGED_PAGES = 2048;  // page ids of a tile's keys that are staged in LDS
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

// what a lane holds of an operand: four consecutive elements
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

template <typename T>
__device__ inline typename Quad<T>::type ld_quad(const T* p) {
    return *reinterpret_cast<const typename Quad<T>::type*>(p);
}

// acc[16 x 16] += A[16 x 4 quads] B[4 quads x 16]: float32 in four instructions of one element
// a lane each, bfloat16 in one instruction of four
__device__ inline f32x4 mma(f32x4 a, f32x4 b, f32x4 acc) {
#pragma unroll
    for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j], b[j], acc, 0, 0, 0);
    return acc;
}
__device__ inline f32x4 mma(s16x4 a, s16x4 b, f32x4 acc) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, acc, 0, 0, 0);
}

__device__ inline void to_quad(const f32x4& p, f32x4& out) { out = p; }
__device__ inline void to_quad(const f32x4& p, s16x4& out) {
    // the hardware's conversion (round to nearest even), two elements an instruction
    typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
    bf16x4 b;
#pragma unroll
    for (int i = 0; i < 4; ++i) b[i] = (__bf16)p[i];
    out = __builtin_bit_cast(s16x4, b);
}
__device__ inline float quad_elem(const f32x4& q, int i) { return q[i]; }
__device__ inline void store_quad(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
__device__ inline void store_quad(bf16_t* p, f32x4 v) {
    s16x4 o;
    to_quad(v, o);
    *reinterpret_cast<s16x4*>(p) = o;
}

// exponentials: float32 keeps the library's; bfloat16 works in powers of two (the scores are
// multiplied by scale * log2(e)) on the hardware's instruction
template <typename T>
__device__ inline float fexp(float x);
template <>
__device__ inline float fexp<float>(float x) {
    return expf(x);
}
template <>
__device__ inline float fexp<bf16_t>(float x) {
    return __builtin_amdgcn_exp2f(x);
}
// tanh of a capped score: the library's in float32; in bfloat16 1 - 2 / (1 + e^(2x)) on the
// hardware's exponential and reciprocal (exact at both ends: e^(2x) = inf gives 1, 0 gives -1)
template <typename T>
__device__ inline float ftanh(float x);
template <>
__device__ inline float ftanh<float>(float x) {
    return tanhf(x);
}
template <>
__device__ inline float ftanh<bf16_t>(float x) {
    return 1.f - 2.f * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(2.8853900817779268f * x));
}

// the four lanes (r, g = 0..3) that share a row: the same bits in each of them.  Two lane swaps
// of gfx950 (the halves of the wave, then neighbouring rows of 16) instead of two trips through
// the LDS crossbar; maximum and sum are commutative, so both partners of a swap get the same bits.
__device__ inline float row_max(float v) {
    const unsigned u = __float_as_uint(v);
    const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const unsigned w = __float_as_uint(fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1])));
    const auto b = __builtin_amdgcn_permlane16_swap(w, w, false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ inline float row_sum(float v) {
    const unsigned u = __float_as_uint(v);
    const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const unsigned w = __float_as_uint(__uint_as_float(a[0]) + __uint_as_float(a[1]));
    const auto b = __builtin_amdgcn_permlane16_swap(w, w, false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// tile_info: [tiles][3] = index of the request's first token in the step, its tokens in the
// step, first row of the tile.  The request's first position is read from `positions`.
// A workgroup's tile is R blocks of 16 rows: every wave multiplies a key tile it has read with
// all R blocks in turn, so that what is read from the cache serves R times the rows (a step of
// portions is bound by those reads).  A row's sums do not depend on R.
template <typename T, int AW, int R>
__global__ __launch_bounds__(AW* RL_WAVE) void attn_tile_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    T* __restrict__ out, const int* __restrict__ tile_info, const int* __restrict__ positions,
    const int* __restrict__ token_slot, const int* __restrict__ block_table, int table_stride,
    int page_size, int nq, int nkv, int window, int keep_first, int sink, float scale,
    float* __restrict__ part, int nsplit, const float* __restrict__ sink_values, float cap,
    const float* __restrict__ slopes) {
    typedef typename Quad<T>::type quad;
    const float in_log2 = sizeof(T) == 2 ? 1.4426950408889634f : 1.f;  // bfloat16: scores in units of log2
    const float cap_in = cap > 0.f ? scale / cap : 0.f;  // a raw product times this is s / cap
    const float cap_out = cap * in_log2;
    const bool adjusted = cap > 0.f || slopes != nullptr;
    scale *= in_log2;
    const int tile = blockIdx.x;
    const int hk = blockIdx.y;
    const int G = nq / nkv;
    const int at = tile_info[3 * tile], n = tile_info[3 * tile + 1], row0 = tile_info[3 * tile + 2];
    __shared__ float fold_ml[AW - 1][R][2][RL_WAVE];
    __shared__ float fold_acc[AW - 1][R][VB * 4][RL_WAVE];
    const int lane = threadIdx.x & (RL_WAVE - 1);
    const int wave = threadIdx.x / RL_WAVE;
    const int r16 = lane & 15;
    const int g = lane >> 4;
    const int start = positions[at];
    const int* table = block_table + (size_t)token_slot[at] * table_stride;

    const int rows = n * G;
    const int keep = window > 0 ? keep_first : 0;  // keys below it are seen from anywhere
    bool row_ok[R];
    int tok[R], head[R], kend[R], kstart[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int row = row0 + 16 * r + r16;
        row_ok[r] = row < rows;
        tok[r] = (row_ok[r] ? row : rows - 1) / G;
        head[r] = hk * G + (row_ok[r] ? row : rows - 1) % G;
        const int pos = start + tok[r];
        kend[r] = pos + 1;
        kstart[r] = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    }
    float slope[R];  // what a position of distance costs this lane's row, in the scores' unit
#pragma unroll
    for (int r = 0; r < R; ++r) slope[r] = slopes ? slopes[head[r]] * in_log2 : 0.f;
    // a raw product of row r and key `key` as the softmax takes it
    auto scored = [&](float raw, int key, int r) -> float {
        if (!adjusted) return raw * scale;
        const float v = cap > 0.f ? cap_out * ftanh<T>(raw * cap_in) : raw * scale;
        return v - slope[r] * (float)(kend[r] - 1 - key);
    };
    const int blocks = min(R, (rows - row0 + 15) / 16);  // blocks of the tile that hold rows
    // keys [all_lo, all_hi) are seen by every row of a block (none where the block is not full):
    // a tile of keys inside needs no masks
    int all_lo[R], all_hi[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int rf = row0 + 16 * r, rl = rf + 15;
        all_lo[r] = 1;
        all_hi[r] = 0;
        if (rl < rows) {
            const int pl = start + rl / G;
            all_hi[r] = start + rf / G + 1;
            all_lo[r] = (window > 0 && pl - window + 1 > 0) ? pl - window + 1 : 0;
        }
    }

    // the keys any row of the tile sees: the kept first ones, and from the first row's first key
    // (rows ascend with the tokens), in whole tiles of 16, up to the last row's own position
    const int first_pos = start + row0 / G;
    const int last_pos = start + (min(rows, row0 + 16 * R) - 1) / G;
    const int first_key = (window > 0 && first_pos - window + 1 > 0) ? first_pos - window + 1 : 0;
    const int lo = first_key & ~15;
    const int hi = last_pos + 1;                     // keys below hi are in the cache
    const int kept_end = min((keep + 15) & ~15, lo);  // tiles [0, kept_end) come before those of [lo, hi)

    // The page ids of both runs of keys, staged once: a step then waits for its keys and values
    // alone, not for a table entry first.  A tile with more pages than fit reads the table itself.
    __shared__ int s_pages[MAX_STAGED_PAGES];
    const int kept_pages = (kept_end + page_size - 1) / page_size;
    const int lo_page = lo / page_size;
    const int late_pages = (hi + page_size - 1) / page_size - lo_page;
    const bool staged = kept_pages + late_pages <= MAX_STAGED_PAGES;
    if (staged) {
        for (int i = threadIdx.x; i < kept_pages + late_pages; i += AW * RL_WAVE)
            s_pages[i] = table[i < kept_pages ? i : lo_page + (i - kept_pages)];
        __syncthreads();
    }
    auto page_of = [&](int key) -> int {
        const int idx = key / page_size;
        if (!staged) return table[idx];
        return s_pages[idx >= lo_page ? kept_pages + (idx - lo_page) : idx];
    };

    // Q^T: lane (row r16, g) holds channels 16c + 4g .. + 3 of its row of every block
    quad qf[R][DB];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const T* qrow = q + ((size_t)(at + tok[r]) * nq + head[r]) * D + 4 * g;
#pragma unroll
        for (int c = 0; c < DB; ++c) {
            qf[r][c] = ld_quad<T>(qrow + 16 * c);
            if (!row_ok[r]) {
#pragma unroll
                for (int i = 0; i < 4; ++i) qf[r][c][i] = 0;
            }
        }
    }

    float m[R], l[R];
    f32x4 acc[R][VB];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        m[r] = -INFINITY;
        l[r] = 0.f;
#pragma unroll
        for (int b = 0; b < VB; ++b) acc[r][b] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }

    // operands of one tile of 16 keys: lane (key r16, g) reads channels 16c + 4g .. + 3 of its
    // key; lane (channel r16, g) reads keys kb + 4g .. + 3 of its channel in every block
    struct Frags {
        quad k[DB], v[VB];
    };
    auto load = [&](int kb, Frags& f) {
        const int key = min(kb + r16, hi - 1);  // beyond the cache: any real key, masked below
        const T* krow =
            k_cache + (((size_t)page_of(key) * nkv + hk) * page_size + key % page_size) * D + 4 * g;
#pragma unroll
        for (int c = 0; c < DB; ++c) f.k[c] = ld_quad<T>(krow + 16 * c);
        const int key4 = min(kb + 4 * g, (hi - 1) & ~3);
        const T* vrow = v_cache + (((size_t)page_of(key4) * nkv + hk) * DV + r16) * page_size +
                        key4 % page_size;
#pragma unroll
        for (int b = 0; b < VB; ++b) f.v[b] = ld_quad<T>(vrow + (size_t)16 * b * page_size);
    };

    // S^T = K Q^T of one tile and one block of rows, the chunks dealt to four accumulators that
    // are added at the end (one chain of dependent instructions would leave the matrix core idle)
    auto scores = [&](const Frags& f, int r) -> f32x4 {
        f32x4 part[4];
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) part[a4] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < DB; ++c) part[c & 3] = mma(f.k[c], qf[r][c], part[c & 3]);
        return (part[0] + part[1]) + (part[2] + part[3]);
    };

    // softmax and second product of the tile at kb for block r, given its scores and its values
    auto finish_block = [&](int kb, int r, f32x4 s, const quad (&vcur)[VB]) {
        // ---- this lane's keys kb + 4g + i of its own row ------------------------------------
        float tmax = -INFINITY;
        if (kb >= all_lo[r] && kb + 16 <= all_hi[r]) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                s[i] = scored(s[i], kb + 4 * g + i, r);
                tmax = fmaxf(tmax, s[i]);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = kb + 4 * g + i;
                const bool seen = row_ok[r] && key < kend[r] && (key >= kstart[r] || key < keep);
                s[i] = seen ? scored(s[i], key, r) : -INFINITY;
                tmax = fmaxf(tmax, s[i]);
            }
        }
        tmax = row_max(tmax);
        const float m_new = fmaxf(m[r], tmax);
        float alpha = 1.f;  // no visible key so far and none here: nothing changes
        f32x4 p = (f32x4){0.f, 0.f, 0.f, 0.f};
        if (m_new != -INFINITY) {
            alpha = fexp<T>(m[r] - m_new);  // m = -inf before the row's first key: 0
#pragma unroll
            for (int i = 0; i < 4; ++i) p[i] = fexp<T>(s[i] - m_new);  // masked: exactly 0
        }
        l[r] = l[r] * alpha + row_sum((p[0] + p[1]) + (p[2] + p[3]));
        m[r] = m_new;
        quad pq;
        to_quad(p, pq);
        // ---- O^T = O^T alpha + V^T P^T --------------------------------------------------------
#pragma unroll
        for (int b = 0; b < VB; ++b) {
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[r][b][i] *= alpha;
            acc[r][b] = mma(vcur[b], pq, acc[r][b]);
        }
    };
    // keys no row of the tile sees (beyond the cache, or between the kept ones and the window,
    // whose pages may have been given back) may hold anything: 0 * it must be 0
    auto clean = [&](int kb, quad (&v)[VB]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = kb + 4 * g + i;
            if (key >= hi || (key < first_key && key >= keep)) {
#pragma unroll
                for (int b = 0; b < VB; ++b) v[b][i] = 0;
            }
        }
    };

    // The wave's tiles, in ascending order: those of the kept keys with index % units == unit,
    // then those of [lo, hi) with index % units == unit.  A launch may deal a tile's keys to
    // several workgroups (blockIdx.z of nsplit): the units are then all their waves.
    const int units = AW * nsplit;
    const int unit = blockIdx.z * AW + wave;
    const int STEP = 16 * units;
    const int kept_mine = 16 * unit;
    const int kept_tiles = kept_mine < kept_end ? (kept_end - kept_mine + STEP - 1) / STEP : 0;
    const int mine = lo + 16 * (((unit - lo / 16) % units + units) % units);  // first tile >= lo with index % units == unit
    const int late_tiles = mine < hi ? (hi - mine + STEP - 1) / STEP : 0;
    const int total = kept_tiles + late_tiles;
    auto kb_of = [&](int i) -> int {
        return i < kept_tiles ? kept_mine + i * STEP : mine + (i - kept_tiles) * STEP;
    };
    if constexpr (R == 1) {
        // Software pipeline over the wave's tiles: while a tile goes through softmax and the
        // second product, the scores of the next have been multiplied and the operands of the one
        // after are in flight.  The last two tiles stand outside the loop, so that inside it the
        // loads are issued without a condition.
        if (total > 0) {
            int left = total;  // tiles of this wave, the current one included
            int i = 0;
            Frags nxt;
            quad vcur[VB], vnext[VB];
            load(kb_of(0), nxt);
            f32x4 sc = scores(nxt, 0);
#pragma unroll
            for (int b = 0; b < VB; ++b) vcur[b] = nxt.v[b];
            if (left > 1) load(kb_of(1), nxt);
            while (left > 2) {
                const f32x4 s_next = scores(nxt, 0);
#pragma unroll
                for (int b = 0; b < VB; ++b) vnext[b] = nxt.v[b];
                load(kb_of(i + 2), nxt);
                __builtin_amdgcn_sched_barrier(0);
                clean(kb_of(i), vcur);
                finish_block(kb_of(i), 0, sc, vcur);
                sc = s_next;
#pragma unroll
                for (int b = 0; b < VB; ++b) vcur[b] = vnext[b];
                ++i;
                --left;
            }
            if (left == 2) {
                const f32x4 s_next = scores(nxt, 0);
                clean(kb_of(i), vcur);
                finish_block(kb_of(i), 0, sc, vcur);
                clean(kb_of(i + 1), nxt.v);
                finish_block(kb_of(i + 1), 0, s_next, nxt.v);
            } else {
                clean(kb_of(i), vcur);
                finish_block(kb_of(i), 0, sc, vcur);
            }
        }
    } else {
        // several blocks of rows: the next tile's operands travel while this one is multiplied
        // with every block in turn
        if (total > 0) {
            Frags cur, nxt;
            load(kb_of(0), cur);
            for (int i = 0; i < total; ++i) {
                const int kb = kb_of(i);
                load(kb_of(min(i + 1, total - 1)), nxt);  // the last one again: no load behind a condition
                __builtin_amdgcn_sched_barrier(0);
                clean(kb, cur.v);
#pragma unroll
                for (int r = 0; r < R; ++r)
                    if (r < blocks) finish_block(kb, r, scores(cur, r), cur.v);
                cur = nxt;
            }
        }
    }
    // ---- fold the waves' states in their order (a wave without visible keys has m = -inf,
    // l = 0 and zero sums: it changes nothing, exactly) ----------------------------------------
    if (wave > 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            fold_ml[wave - 1][r][0][lane] = m[r];
            fold_ml[wave - 1][r][1][lane] = l[r];
#pragma unroll
            for (int b = 0; b < VB; ++b)
#pragma unroll
                for (int i = 0; i < 4; ++i) fold_acc[wave - 1][r][4 * b + i][lane] = acc[r][b][i];
        }
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int w = 0; w < AW - 1; ++w) {
            const float m_w = fold_ml[w][r][0][lane], l_w = fold_ml[w][r][1][lane];
            const float m_new = fmaxf(m[r], m_w);
            if (m_new == -INFINITY) continue;
            const float fa = fexp<T>(m[r] - m_new), fb = fexp<T>(m_w - m_new);
            l[r] = l[r] * fa + l_w * fb;
#pragma unroll
            for (int b = 0; b < VB; ++b)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    acc[r][b][i] = acc[r][b][i] * fa + fold_acc[w][r][4 * b + i][lane] * fb;
            m[r] = m_new;
        }
        if (!row_ok[r]) continue;
        if (nsplit > 1) {
            // this workgroup's share of the row's keys: sums, maximum and denominator go to the
            // merge kernel as they are
            float* prow = part + (((size_t)(at + tok[r]) * nq + head[r]) * nsplit + blockIdx.z) * (DV + 2);
#pragma unroll
            for (int b = 0; b < VB; ++b) *reinterpret_cast<f32x4*>(prow + 16 * b + 4 * g) = acc[r][b];
            if (g == 0) {
                prow[DV] = m[r];
                prow[DV + 1] = l[r];
            }
            continue;
        }
        // the key of score 0 that has no value: exp(0 - m) more in the denominator; with
        // `sink_values` its score is a number of the row's head (not scaled), which may lie
        // above every real score: the state is brought to the larger maximum first
        if (sink) {
            float s0 = 0.f;
            if (sink_values) {
                s0 = sink_values[head[r]];
                if constexpr (sizeof(T) == 2) s0 *= 1.4426950408889634f;
            }
            const float m_new = fmaxf(m[r], s0);
            const float fa = fexp<T>(m[r] - m_new);
            l[r] = l[r] * fa + fexp<T>(s0 - m_new);
#pragma unroll
            for (int b = 0; b < VB; ++b)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[r][b][i] *= fa;
        }
        // acc[r][b][i] is channel 16b + 4g + i of the lane's row
        T* orow = out + ((size_t)(at + tok[r]) * nq + head[r]) * DV + 4 * g;
        const float inv = 1.f / l[r];
#pragma unroll
        for (int b = 0; b < VB; ++b)
            store_quad(orow + 16 * b, (f32x4){acc[r][b][0] * inv, acc[r][b][1] * inv, acc[r][b][2] * inv,
                                              acc[r][b][3] * inv});
    }
}

// Fold the shares of a row's keys that nsplit (at most 64) workgroups left, in order (the same
// bits every run), add the sink's term and write the row.  One wave a row: lane s holds share s's
// maximum and sum, every lane takes them from there, and a lane's channels are read eight shares
// at a time so that the reads of a channel are in flight together.
__global__ __launch_bounds__(256) void attn_tile_merge_kernel(const float* __restrict__ part,
                                                              bf16_t* __restrict__ out, int rows, int nsplit,
                                                              int sink, const float* __restrict__ sink_values,
                                                              int nq) {
    const int row = blockIdx.x * 4 + threadIdx.x / RL_WAVE;
    const int lane = threadIdx.x & (RL_WAVE - 1);
    if (row >= rows) return;
    const float* p = part + (size_t)row * nsplit * (DV + 2);
    const bool mine = lane < nsplit;
    const float m = mine ? p[lane * (DV + 2) + DV] : -INFINITY;
    const float l = mine ? p[lane * (DV + 2) + DV + 1] : 0.f;
    float top = m;
#pragma unroll
    for (int off = RL_WAVE / 2; off > 0; off >>= 1) top = fmaxf(top, __shfl_xor(top, off));
    // the sink's score: 0, or a number of the row's head (rows are (token, head) pairs)
    const float s0 = (sink && sink_values) ? sink_values[row % nq] * 1.4426950408889634f : 0.f;
    if (sink) top = fmaxf(top, s0);
    const float weight = mine ? __builtin_amdgcn_exp2f(m - top) : 0.f;
    float den = 0.f;
    for (int s = 0; s < nsplit; ++s) den += __shfl(weight, s) * __shfl(l, s);
    if (sink) den += __builtin_amdgcn_exp2f(s0 - top);
    for (int c0 = 0; c0 < DV; c0 += RL_WAVE) {
        const int c = c0 + lane;
        const bool live = c < DV;
        float sum = 0.f;
        for (int s8 = 0; s8 < nsplit; s8 += 8) {
            float v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = (live && s8 + j < nsplit) ? p[(s8 + j) * (DV + 2) + c] : 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) sum += __shfl(weight, (s8 + j) & (RL_WAVE - 1)) * v[j];
        }
        if (live) out[(size_t)row * DV + c] = float_to_bf16(sum / den);
    }
}

}  // namespace tileattn

extern "C" int rl_attn_tile_head_dim() { return tileattn::D; }
extern "C" int rl_attn_tile_value_dim() { return tileattn::DV; }

// Every token of the step, single tokens and portions alike.  page_size must be a multiple
// of 4 (the four keys of a lane lie in one page).
// rows of a workgroup's tile in a bfloat16 launch of portions (tile_rows > 16)
extern "C" int rl_attn_tile_wide_rows() { return 16 * tileattn::PORTION_BLOCKS; }

// Every token of the step, single tokens and portions alike.  page_size must be a multiple
// of 4 (the four keys of a lane lie in one page).  tile_rows: the rows of a tile of tile_info,
// 16 or, in bfloat16, rl_attn_tile_wide_rows().
extern "C" int rl_attn_tile(const void* q, const void* k_cache, const void* v_cache, void* out,
                            const int* tile_info, int num_tiles, const int* positions,
                            const int* token_slot, const int* block_table, int table_stride,
                            int page_size, int nq, int nkv, int window, int keep_first, int sink,
                            float scale, int nsplit, float* part, int tokens, int tile_rows, int act_type,
                            const float* sink_values, float cap, const float* slopes, hipStream_t stream) {
    if (num_tiles <= 0) return RL_OK;
    if (cap < 0.f) return RL_ERR_ARG;
    if (nkv < 1 || nq % nkv || page_size < 4 || page_size % 4 || nkv > 65535 || window < 0 || keep_first < 0)
        return RL_ERR_ARG;
    constexpr int AW = 4;
    constexpr int PB = tileattn::PORTION_BLOCKS;
    dim3 grid(num_tiles, nkv), block(AW * RL_WAVE);
#define RL_TILE_ARGS(TYPE)                                                                                  \
    (const TYPE*)q, (const TYPE*)k_cache, (const TYPE*)v_cache, (TYPE*)out, tile_info, positions, token_slot, \
        block_table, table_stride, page_size, nq, nkv, window, keep_first, sink, scale
    if (act_type == RL_BF16 && tile_rows == 16 * PB && PB > 1) {
        if (nsplit != 1) return RL_ERR_ARG;
        hipLaunchKernelGGL((tileattn::attn_tile_kernel<bf16_t, AW, PB>), grid, block, 0, stream, RL_TILE_ARGS(bf16_t),
                           nullptr, 1, sink_values, cap, slopes);
        return rl_launch_status();
    }
    if (tile_rows != 16) return RL_ERR_ARG;
    // nsplit > 1 (bfloat16 only: the order of the sums changes with it): a launch of few tiles
    // over many keys (single tokens) deals every tile's keys to nsplit workgroups, whose shares
    // the merge kernel folds; a compute unit's load path, not a wave's latency, bounds a tile
    if (nsplit > 1) {
        if (act_type != RL_BF16 || !part || nsplit > 64 || tokens < 1) return RL_ERR_ARG;
        hipLaunchKernelGGL((tileattn::attn_tile_kernel<bf16_t, AW, 1>), dim3(num_tiles, nkv, nsplit), block, 0, stream,
                           RL_TILE_ARGS(bf16_t), part, nsplit, sink_values, cap, slopes);
        const int rows = tokens * nq;
        hipLaunchKernelGGL(tileattn::attn_tile_merge_kernel, dim3((rows + 3) / 4), dim3(256), 0, stream, part,
                           (bf16_t*)out, rows, nsplit, sink, sink_values, nq);
        return rl_launch_status();
    }
    if (act_type == RL_F32)
        hipLaunchKernelGGL((tileattn::attn_tile_kernel<float, AW, 1>), grid, block, 0, stream, RL_TILE_ARGS(float),
                           nullptr, 1, sink_values, cap, slopes);
    else if (act_type == RL_BF16)
        hipLaunchKernelGGL((tileattn::attn_tile_kernel<bf16_t, AW, 1>), grid, block, 0, stream, RL_TILE_ARGS(bf16_t),
                           nullptr, 1, sink_values, cap, slopes);
    else
        return RL_ERR_ARG;
#undef RL_TILE_ARGS
    return rl_launch_status();
}
