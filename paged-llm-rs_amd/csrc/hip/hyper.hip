// Several copies of the residual stream, and experts chosen by a table over token ids.
//
// Copies of the stream.  A model keeps S copies x_1 .. x_S of every row, [n, S, W] in 32-bit.  A sublayer
// reads u = sum_s in[s] x_s through a norm, and its output y rebuilds every copy from all of them:
// x_t <- sum_s mix[s, t] x_s + out[t] y.  One kernel does the rebuild behind one sublayer and the read-out
// (with its norm) in front of the next, a row a workgroup, so that the copies travel once: either half
// may be left out.  Sums, statistic and gain are 32-bit; the normed row is rounded once, when stored.
//
// Experts by table.  Row t uses the `top` experts that table[id of t] names, each weighted 1/top; an
// expert is down(act(gate x) * (up x)).  Two ways.  moe_rows, a workgroup a (row, choice): a row reads its
// own experts' weights, in any type and size (the 32-bit path, and shapes the matrix cores' tiles do not
// take).  moe_sort and moe_combine around the grouped tiled product (gemm_tiled.hip): the step's (row,
// choice) pairs are dealt to their experts, every expert's pairs in tiles of 128 rows, so that an expert's
// weights are read once a tile and multiplied on the matrix cores; a pair's result does not depend on which
// other pairs share its tile.
#include "common.hpp"

#define HC_MAX_COPIES 8

struct HcArgs {
    float* streams;        // [n, S, W]
    const float* y;        // [n, W], or null: the copies stay as they are
    const float* mix;      // [S, S], from x to: with y
    const float* out;      // [S]: with y
    const float* in;       // [S], or null: nothing is read out
    const void* gain;      // [W] 32-bit, or null: the weighted sum as it is
    float eps;
    void* read;            // [rows, W]: the read-out
    const int* rows;       // which rows are read out, or null for all (with a list nothing is rebuilt)
    int S, W;
};

// VEC: how many neighbouring columns a thread takes at a time (4: every load and store is 16 bytes, and a row of
// up to 4,096 values is one round of loads for a workgroup of 1,024 threads, all of them asked for at once).
template <typename T, int VEC>
__global__ __launch_bounds__(1024) void hc_step_kernel(HcArgs a) {
    extern __shared__ float hc_row[];                 // the read-out's row before its norm, then 16 floats of scratch
    float* scratch = hc_row + a.W;
    const int i = blockIdx.x;
    const int r = a.rows != nullptr ? a.rows[i] : i;
    const int S = a.S, W = a.W;
    float* x = a.streams + static_cast<size_t>(r) * S * W;
    const float* y = a.y != nullptr ? a.y + static_cast<size_t>(r) * W : nullptr;
    // The weights travel through LDS: the first eighty threads ask for one of them each, all at once
    // (read one after the other from where they lie, each behind a condition, they were eighty trips to memory in a row).
    __shared__ float hc_w[HC_MAX_COPIES * HC_MAX_COPIES + 2 * HC_MAX_COPIES];
    for (int k = threadIdx.x; k < HC_MAX_COPIES * HC_MAX_COPIES + 2 * HC_MAX_COPIES; k += blockDim.x) {
        if (k < HC_MAX_COPIES * HC_MAX_COPIES) {
            const int s = k / HC_MAX_COPIES, t = k % HC_MAX_COPIES;
            hc_w[k] = (y != nullptr && s < S && t < S) ? a.mix[s * S + t] : 0.f;
        } else if (k < HC_MAX_COPIES * HC_MAX_COPIES + HC_MAX_COPIES) {
            const int t = k - HC_MAX_COPIES * HC_MAX_COPIES;
            hc_w[k] = (y != nullptr && t < S) ? a.out[t] : 0.f;
        } else if (k < HC_MAX_COPIES * HC_MAX_COPIES + 2 * HC_MAX_COPIES) {
            const int t = k - HC_MAX_COPIES * HC_MAX_COPIES - HC_MAX_COPIES;
            hc_w[k] = (a.in != nullptr && t < S) ? a.in[t] : 0.f;
        }
    }
    __syncthreads();
    // (the same for every lane: kept in scalar registers)
    auto uniform = [&](int k) { return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(hc_w[k]))); };
    float mix[HC_MAX_COPIES * HC_MAX_COPIES], out[HC_MAX_COPIES], in[HC_MAX_COPIES];
#pragma unroll
    for (int k = 0; k < HC_MAX_COPIES * HC_MAX_COPIES; ++k) mix[k] = uniform(k);
#pragma unroll
    for (int k = 0; k < HC_MAX_COPIES; ++k) {
        out[k] = uniform(HC_MAX_COPIES * HC_MAX_COPIES + k);
        in[k] = uniform(HC_MAX_COPIES * HC_MAX_COPIES + HC_MAX_COPIES + k);
    }
    typedef float vec_t __attribute__((ext_vector_type(VEC)));
    float ss = 0.f;
    for (int c = threadIdx.x * VEC; c < W; c += blockDim.x * VEC) {
        vec_t v[HC_MAX_COPIES];
#pragma unroll
        for (int s = 0; s < HC_MAX_COPIES; ++s) {
            if (s < S) v[s] = *reinterpret_cast<const vec_t*>(x + static_cast<size_t>(s) * W + c);
            else v[s] = vec_t(0.f);
        }
        if (y != nullptr) {
            const vec_t add = *reinterpret_cast<const vec_t*>(y + c);
            vec_t nv[HC_MAX_COPIES];
#pragma unroll
            for (int t = 0; t < HC_MAX_COPIES; ++t) {
                vec_t acc = vec_t(0.f);
#pragma unroll
                for (int s = 0; s < HC_MAX_COPIES; ++s)
                    if (s < S) {
#pragma unroll
                        for (int e = 0; e < VEC; ++e) acc[e] = fmaf(mix[s * HC_MAX_COPIES + t], v[s][e], acc[e]);
                    }
#pragma unroll
                for (int e = 0; e < VEC; ++e) nv[t][e] = fmaf(out[t], add[e], acc[e]);
            }
#pragma unroll
            for (int t = 0; t < HC_MAX_COPIES; ++t) {
                v[t] = nv[t];
                if (t < S) *reinterpret_cast<vec_t*>(x + static_cast<size_t>(t) * W + c) = nv[t];
            }
        }
        if (a.in != nullptr) {
            vec_t u = vec_t(0.f);
#pragma unroll
            for (int s = 0; s < HC_MAX_COPIES; ++s)
                if (s < S) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) u[e] = fmaf(in[s], v[s][e], u[e]);
                }
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                hc_row[c + e] = u[e];
                ss += u[e] * u[e];
            }
        }
    }
    if (a.in == nullptr) return;
    T* o = static_cast<T*>(a.read) + static_cast<size_t>(i) * W;
    if (a.gain == nullptr) {
        // (every thread reads back what it wrote itself)
        for (int c = threadIdx.x * VEC; c < W; c += blockDim.x * VEC)
#pragma unroll
            for (int e = 0; e < VEC; ++e) o[c + e] = from_float<T>(hc_row[c + e]);
        return;
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.f / sqrtf(ss / static_cast<float>(W) + a.eps);
    const float* gain = static_cast<const float*>(a.gain);
    for (int c = threadIdx.x * VEC; c < W; c += blockDim.x * VEC)
#pragma unroll
        for (int e = 0; e < VEC; ++e) o[c + e] = from_float<T>(hc_row[c + e] * inv * gain[c + e]);
}

// streams [n, S, W] (32-bit) in place.  y, mix, out: the rebuild behind a sublayer (all null: none).  in: the
// read-out's weights (null: none); gain (32-bit [W]) and eps: its norm (gain null: no norm); read: [rows, W] in
// `dtype`.  rows: the rows that are read out (null: all n); with a list there is no rebuild.
extern "C" int pl_hc_step(float* streams, const float* y, const float* mix, const float* out, const float* in,
                          const float* gain, float eps, void* read, int dtype, const int* rows, int count, int S, int W,
                          hipStream_t stream) {
    PL_REQUIRE(count >= 0 && S >= 1 && S <= HC_MAX_COPIES && W > 0 && W <= 16368, "hc_step: %d rows of %d copies of %d",
               count, S, W);
    PL_REQUIRE((y == nullptr) == (mix == nullptr) && (y == nullptr) == (out == nullptr),
               "hc_step: a rebuild needs the sublayer's output and both sets of weights");
    PL_REQUIRE(rows == nullptr || y == nullptr, "hc_step: a list of rows and a rebuild");
    PL_REQUIRE((in == nullptr) == (read == nullptr), "hc_step: a read-out needs its weights and its place");
    if (count == 0 || (y == nullptr && in == nullptr)) return 0;
    HcArgs a{streams, y, mix, out, in, gain, eps, read, rows, S, W};
    const size_t lds = (static_cast<size_t>(W) + 16) * sizeof(float);
    PL_REQUIRE(dtype == PL_DTYPE_F32 || dtype == PL_DTYPE_BF16, "hc_step: dtype code %d", dtype);
    if (W % 4 == 0) {
        // a thread a quad of columns, one round of loads up to a width of 4,096
        int threads = ((W / 4 + 63) / 64) * 64;
        threads = threads > 1024 ? 1024 : threads;
        if (dtype == PL_DTYPE_F32) hc_step_kernel<float, 4><<<count, threads, lds, stream>>>(a);
        else hc_step_kernel<bf16_t, 4><<<count, threads, lds, stream>>>(a);
    } else {
        const int threads = W >= 1024 ? 256 : (W >= 256 ? 128 : 64);
        if (dtype == PL_DTYPE_F32) hc_step_kernel<float, 1><<<count, threads, lds, stream>>>(a);
        else hc_step_kernel<bf16_t, 1><<<count, threads, lds, stream>>>(a);
    }
    PL_CHECK_LAUNCH("hc_step");
    return 0;
}

__global__ void stream_copies_kernel(const float* __restrict__ x, float* __restrict__ out, int S, int W) {
    const size_t t = blockIdx.x;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float v = x[t * W + c];
        for (int s = 0; s < S; ++s) out[(t * S + s) * W + c] = v;
    }
}

// out[t, s, :] = x[t, :] for every s
extern "C" int pl_stream_copies(const float* x, float* out, int n, int S, int W, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && S >= 1 && W > 0, "stream_copies: %d rows, %d copies of %d", n, S, W);
    if (n == 0) return 0;
    stream_copies_kernel<<<n, 256, 0, stream>>>(x, out, S, W);
    PL_CHECK_LAUNCH("stream_copies");
    return 0;
}

__global__ void softcap_kernel(float* __restrict__ x, float cap, size_t count) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < count) x[i] = cap * tanhf(x[i] / cap);
}

// x = cap * tanh(x / cap)
extern "C" int pl_softcap(float* x, float cap, long count, hipStream_t stream) {
    PL_REQUIRE(count >= 0 && cap > 0.f, "softcap: %ld values, a cap of %g", count, static_cast<double>(cap));
    if (count == 0) return 0;
    softcap_kernel<<<static_cast<unsigned>((count + 255) / 256), 256, 0, stream>>>(x, cap, static_cast<size_t>(count));
    PL_CHECK_LAUNCH("softcap");
    return 0;
}

// ---- experts by table, few rows -------------------------------------------------------------------------

// The id of row t: its own, or the one an earlier kernel left on the device (as the embedding takes it).
__device__ __forceinline__ int moe_token(const int* ids, const int* src, const int* fed, int t) {
    int id = ids[t];
    if (src != nullptr) {
        const int from = src[t];
        if (from >= 0) id = fed[from];
    }
    return id;
}

// A wave's dot product of a weight row with a row of 32-bit values in LDS; every lane gets the sum.
// The order of the additions depends on K alone.
template <typename T>
__device__ __forceinline__ float moe_dot(const T* __restrict__ w, const float* xs, int K, int lane) {
    float acc = 0.f;
    if (sizeof(T) == 2 && K % 8 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0) {
        for (int k = lane * 8; k < K; k += 64 * 8) {
            const uint4 raw = *reinterpret_cast<const uint4*>(w + k);
            const uint32_t word[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc = fmaf(__uint_as_float(word[j] << 16), xs[k + 2 * j], acc);
                acc = fmaf(__uint_as_float(word[j] & 0xffff0000u), xs[k + 2 * j + 1], acc);
            }
        }
    } else {
        for (int k = lane; k < K; k += 64) acc = fmaf(to_float(w[k]), xs[k], acc);
    }
    return wave_sum(acc);
}

struct MoeArgs {
    const void* x;         // [n, W]
    const int* ids;
    const int* src;
    const int* fed;
    const int* positions;  // rows at position -1 are padding
    const int* table;      // [vocab, top]
    const void* w_gu;      // [E, 2 F, W]: an expert's gate rows, then its up rows
    const void* w_down;    // [E, W, F]
    void* h;               // [n, top, F]
    float* out;            // [n, W]
    int n, W, F, E, top, vocab, act;
    // Where a router has chosen (null: the table decides and every choice counts 1/top): the expert of pair
    // (t, c) is choice[t * top + c], -1 for none, E .. E + identity - 1 for an identity expert, whose output is the
    // row itself; weight[t * top + c] is what the pair counts.
    const int* choice;
    const float* weight;
    int identity;
};

// The expert of pair (t, c), or -1: the router's choice, or the table's row of the token's id.
__device__ __forceinline__ int moe_pair_expert(const MoeArgs& a, int t, int c) {
    if (a.choice != nullptr) return a.choice[static_cast<size_t>(t) * a.top + c];
    const int id = moe_token(a.ids, a.src, a.fed, t);
    if (id < 0 || id >= a.vocab) return -1;
    return a.table[static_cast<size_t>(id) * a.top + c];
}

template <typename T>
__global__ __launch_bounds__(256) void moe_up_kernel(MoeArgs a) {
    extern __shared__ float moe_x[];
    const int t = blockIdx.x / a.top, c = blockIdx.x % a.top;
    if (a.positions[t] < 0) return;
    const int e = moe_pair_expert(a, t, c);
    if (e < 0 || e >= a.E) return;
    const int W = a.W, F = a.F;
    const T* x = static_cast<const T*>(a.x) + static_cast<size_t>(t) * W;
    for (int k = threadIdx.x; k < W; k += blockDim.x) moe_x[k] = to_float(x[k]);
    __syncthreads();
    const int lane = threadIdx.x % PL_WAVE, wave = threadIdx.x / PL_WAVE, waves = blockDim.x / PL_WAVE;
    const T* gate = static_cast<const T*>(a.w_gu) + static_cast<size_t>(e) * 2 * F * W;
    const T* up = gate + static_cast<size_t>(F) * W;
    T* h = static_cast<T*>(a.h) + (static_cast<size_t>(t) * a.top + c) * F;
    for (int f = blockIdx.y * waves + wave; f < F; f += gridDim.y * waves) {
        const float g = moe_dot<T>(gate + static_cast<size_t>(f) * W, moe_x, W, lane);
        const float u = moe_dot<T>(up + static_cast<size_t>(f) * W, moe_x, W, lane);
        if (lane == 0) h[f] = from_float<T>(pl_activate<true>(g, a.act) * u);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(MoeArgs a) {
    extern __shared__ float moe_h[];                  // [top, F]
    const int t = blockIdx.x;
    const int W = a.W, F = a.F, top = a.top;
    float* o = a.out + static_cast<size_t>(t) * W;
    const int lane = threadIdx.x % PL_WAVE, wave = threadIdx.x / PL_WAVE, waves = blockDim.x / PL_WAVE;
    const int id = a.positions[t] < 0 ? -1 : (a.choice != nullptr ? 0 : moe_token(a.ids, a.src, a.fed, t));
    if (id < 0 || id >= a.vocab) {
        for (int w = blockIdx.y * blockDim.x + threadIdx.x; w < W; w += gridDim.y * blockDim.x) o[w] = 0.f;
        return;
    }
    const T* x = static_cast<const T*>(a.x) + static_cast<size_t>(t) * W;
    const T* h = static_cast<const T*>(a.h) + static_cast<size_t>(t) * top * F;
    for (int k = threadIdx.x; k < top * F; k += blockDim.x) moe_h[k] = to_float(h[k]);
    __syncthreads();
    const float share = 1.f / static_cast<float>(top);
    for (int w = blockIdx.y * waves + wave; w < W; w += gridDim.y * waves) {
        float sum = 0.f;
        for (int c = 0; c < top; ++c) {
            const int e = moe_pair_expert(a, t, c);
            const float counts = a.weight != nullptr ? a.weight[static_cast<size_t>(t) * top + c] : share;
            if (e >= a.E && e < a.E + a.identity) sum += to_float(x[w]) * counts;
            if (e < 0 || e >= a.E) continue;
            const T* down = static_cast<const T*>(a.w_down) + (static_cast<size_t>(e) * W + w) * F;
            sum += moe_dot<T>(down, moe_h + c * F, F, lane) * counts;
        }
        if (lane == 0) o[w] = sum;
    }
}

// out[t] (32-bit) = (1/top) sum over the experts e that table[id of t] names of down_e (act(gate_e x_t) * (up_e x_t)).
// x [n, W], w_gu [E, 2 F, W], w_down [E, W, F] and the workspace h [n, top, F] in `dtype`; table [vocab, top].
// With `choice` [n, top] (and `weight` [n, top]) a router has chosen instead of the table: see MoeArgs.
extern "C" int pl_moe_rows(const void* x, const int* ids, const int* src, const int* fed, const int* positions,
                           const int* table, const void* w_gu, const void* w_down, void* h, float* out, int dtype,
                           int n, int W, int F, int E, int top, int vocab, int act, const int* choice, const float* weight,
                           int identity, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && W > 0 && F > 0 && E > 0 && top > 0 && top <= E + identity && identity >= 0 && vocab > 0 && act >= 0 && act <= 2,
               "moe_rows: %d rows of %d, %d experts of %d, %d a row", n, W, E, F, top);
    PL_REQUIRE((choice != nullptr) != (table != nullptr) && (weight == nullptr || choice != nullptr),
               "moe_rows: the experts of a row are a table's or a router's");
    PL_REQUIRE((src == nullptr) == (fed == nullptr), "moe_rows: rows fed from the step before need both the rows and the tokens");
    PL_REQUIRE(W <= 16384 && static_cast<long long>(top) * F <= 16384, "moe_rows: rows of %d, %d experts of %d a row", W, top, F);
    PL_REQUIRE(static_cast<long long>(n) * top < (1ll << 31), "moe_rows: %d rows", n);
    if (n == 0) return 0;
    MoeArgs a{x, ids, src, fed, positions, table, w_gu, w_down, h, out, n, W, F, E, top, vocab, act, choice, weight, identity};
    // few rows: deal an expert's rows of weights to several workgroups, so that the chip has work
    const int cu = pl_compute_units();
    int up_parts = 1, down_parts = 1;
    while (static_cast<long long>(n) * top * up_parts < 2ll * cu && up_parts * 8 < F) up_parts *= 2;
    while (static_cast<long long>(n) * down_parts < 2ll * cu && down_parts * 8 < W) down_parts *= 2;
    const dim3 up_grid(n * top, up_parts), down_grid(n, down_parts);
    if (dtype == PL_DTYPE_F32) {
        moe_up_kernel<float><<<up_grid, 256, W * sizeof(float), stream>>>(a);
        moe_down_kernel<float><<<down_grid, 256, static_cast<size_t>(top) * F * sizeof(float), stream>>>(a);
    } else if (dtype == PL_DTYPE_BF16) {
        moe_up_kernel<bf16_t><<<up_grid, 256, W * sizeof(float), stream>>>(a);
        moe_down_kernel<bf16_t><<<down_grid, 256, static_cast<size_t>(top) * F * sizeof(float), stream>>>(a);
    } else {
        PL_REQUIRE(false, "moe_rows: dtype code %d", dtype);
    }
    PL_CHECK_LAUNCH("moe_rows");
    return 0;
}

// ---- experts by table, the pairs dealt to their experts ---------------------------------------------------------

// One workgroup.  Pair p = t * top + c (row t, its c-th expert).  Expert e's pairs get the slots
// base[e] .. base[e] + count[e] - 1, base[e] a multiple of `tile`; gather[slot] = t (or -1 for the slots
// between the experts' stretches), slot_of[p] = slot (or -1 for a pair of a padding row),
// tile_group[i] = the expert of tile i (or -1 behind the last).  Which of an expert's pairs gets which of
// its slots is left to the order in which the threads arrive: nothing computed from a slot depends on it.
__global__ __launch_bounds__(1024) void moe_sort_kernel(const int* ids, const int* src, const int* fed, const int* positions,
                                                        const int* table, const int* choice, int n, int top, int E, int vocab, int tile,
                                                        int tiles, int* gather, int* slot_of, int* tile_group) {
    extern __shared__ int moe_counts[];               // count [E], base [E], cursor [E]
    int* count = moe_counts;
    int* base = moe_counts + E;
    int* cursor = moe_counts + 2 * E;
    for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = cursor[e] = 0;
    for (int s = threadIdx.x; s < tiles * tile; s += blockDim.x) gather[s] = -1;
    __syncthreads();
    const int pairs = n * top;
    auto expert_of = [&](int p) -> int {
        const int t = p / top;
        if (positions[t] < 0) return -1;
        int e;
        if (choice != nullptr) {
            e = choice[p];                            // (an identity expert, E or beyond, takes no slot)
        } else {
            const int id = moe_token(ids, src, fed, t);
            if (id < 0 || id >= vocab) return -1;
            e = table[static_cast<size_t>(id) * top + (p - t * top)];
        }
        return (e >= 0 && e < E) ? e : -1;
    };
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
        const int e = expert_of(p);
        slot_of[p] = e;                               // (kept for the second pass, which the same thread makes)
        if (e >= 0) atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0;                                   // in tiles
        for (int e = 0; e < E; ++e) {
            base[e] = at * tile;
            const int mine = (count[e] + tile - 1) / tile;
            for (int i = 0; i < mine && at + i < tiles; ++i) tile_group[at + i] = e;
            at += mine;
        }
        for (; at < tiles; ++at) tile_group[at] = -1;
    }
    __syncthreads();
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
        const int e = slot_of[p];
        int slot = -1;
        if (e >= 0) {
            slot = base[e] + atomicAdd(&cursor[e], 1);
            gather[slot] = p / top;
        }
        slot_of[p] = slot;
    }
}

// tiles: what the caller has room for, at least ceil(n * top / tile) + min(E, n * top).
extern "C" int pl_moe_sort(const int* ids, const int* src, const int* fed, const int* positions, const int* table,
                           const int* choice, int n, int top, int E, int vocab, int tile, int tiles, int* gather, int* slot_of,
                           int* tile_group, hipStream_t stream) {
    PL_REQUIRE(n > 0 && top > 0 && E > 0 && E <= 4096 && vocab > 0 && tile > 0, "moe_sort: %d rows, %d of %d experts", n, top, E);
    PL_REQUIRE((choice != nullptr) != (table != nullptr), "moe_sort: the experts of a row are a table's or a router's");
    PL_REQUIRE(static_cast<long long>(n) * top < (1ll << 30) && tiles >= (n * top + tile - 1) / tile + (E < n * top ? E : n * top),
               "moe_sort: %d tiles of %d for %d rows with %d of %d experts", tiles, tile, n, top, E);
    PL_REQUIRE((src == nullptr) == (fed == nullptr), "moe_sort: rows fed from the step before need both the rows and the tokens");
    moe_sort_kernel<<<1, 1024, 3 * E * sizeof(int), stream>>>(ids, src, fed, positions, table, choice, n, top, E, vocab, tile, tiles,
                                                               gather, slot_of, tile_group);
    PL_CHECK_LAUNCH("moe_sort");
    return 0;
}

// out[t, :] = (1/top) sum over c of y[slot_of[t * top + c], :], the choices in their order; a pair without a slot adds nothing.
// y may come in `splits` copies, `split_stride` floats apart, each a stretch of the product's inner width: a pair's
// copies are added in their order.
// With `weight` a pair counts weight[t * top + c] instead of 1/top, and a pair whose `choice` is E or beyond (an
// identity expert) adds the row of x itself (of type `x_dtype`) with its weight.
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ y, const int* __restrict__ slot_of,
                                                          float* __restrict__ out, int top, int W, int splits, size_t split_stride,
                                                          const float* __restrict__ weight, const int* __restrict__ choice,
                                                          const void* __restrict__ x, int x_dtype, int E,
                                                          const int* __restrict__ positions) {
    const int t = blockIdx.x;
    const float even = 1.f / static_cast<float>(top);
    const bool padding = positions != nullptr && positions[t] < 0;        // (a row of padding has no identity expert either)
    for (int w = threadIdx.x * 4; w < W; w += blockDim.x * 4) {
        float4 sum = {0.f, 0.f, 0.f, 0.f};
        for (int c = 0; c < top; ++c) {
            const int slot = slot_of[t * top + c];
            const float share = weight != nullptr ? weight[t * top + c] : even;
            if (slot < 0) {
                if (choice != nullptr && !padding && choice[t * top + c] >= E) {
                    const size_t at = static_cast<size_t>(t) * W + w;
                    sum.x += load_as_float(x, x_dtype, at) * share;
                    sum.y += load_as_float(x, x_dtype, at + 1) * share;
                    sum.z += load_as_float(x, x_dtype, at + 2) * share;
                    sum.w += load_as_float(x, x_dtype, at + 3) * share;
                }
                continue;
            }
            float4 v = *reinterpret_cast<const float4*>(y + static_cast<size_t>(slot) * W + w);
            for (int s = 1; s < splits; ++s) {
                const float4 more = *reinterpret_cast<const float4*>(y + s * split_stride + static_cast<size_t>(slot) * W + w);
                v.x += more.x;
                v.y += more.y;
                v.z += more.z;
                v.w += more.w;
            }
            sum.x += v.x * share;
            sum.y += v.y * share;
            sum.z += v.z * share;
            sum.w += v.w * share;
        }
        *reinterpret_cast<float4*>(out + static_cast<size_t>(t) * W + w) = sum;
    }
}

extern "C" int pl_moe_combine(const float* y, const int* slot_of, float* out, int n, int top, int W, int splits,
                              long long split_stride, const float* weight, const int* choice, const void* x, int x_dtype,
                              int E, const int* positions, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && top > 0 && W > 0 && W % 4 == 0 && splits >= 1, "moe_combine: %d rows of %d, %d a row, %d copies", n, W, top, splits);
    PL_REQUIRE(choice == nullptr || (x != nullptr && (x_dtype == PL_DTYPE_F32 || x_dtype == PL_DTYPE_BF16)),
               "moe_combine: identity experts need the rows they hand through");
    if (n == 0) return 0;
    moe_combine_kernel<<<n, 256, 0, stream>>>(y, slot_of, out, top, W, splits, static_cast<size_t>(split_stride), weight, choice,
                                              x, x_dtype, E, positions);
    PL_CHECK_LAUNCH("moe_combine");
    return 0;
}

// ---- a router's choice ------------------------------------------------------------------------------------

// The lane that holds the largest value (the lowest index among equals) learns nothing special: every lane gets
// (value, index) of the winner.
__device__ __forceinline__ void wave_best(float& v, int& i) {
#pragma unroll
    for (int off = PL_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(v, off, PL_WAVE);
        const int oi = __shfl_xor(i, off, PL_WAVE);
        if (ov > v || (ov == v && oi < i)) {
            v = ov;
            i = oi;
        }
    }
}

// Four dot products of a wave at once, rows e0, e0 + step, ... of w with a row of 32-bit values in LDS, so that the
// loads of all four are on their way together; every lane gets the sums.  A row at or beyond `total` gives 0.
template <typename T>
__device__ __forceinline__ void router_dots(const T* __restrict__ w, const float* xs, int K, int lane, int e0, int step, int total,
                                            float (&out)[4]) {
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    const T* rows[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) rows[j] = w + static_cast<size_t>(e0 + j * step < total ? e0 + j * step : e0) * K;
    if (sizeof(T) == 2 && K % 8 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0) {
        for (int k = lane * 8; k < K; k += 64 * 8) {
            uint4 raw[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) raw[j] = *reinterpret_cast<const uint4*>(rows[j] + k);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t word[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc[j] = fmaf(__uint_as_float(word[i] << 16), xs[k + 2 * i], acc[j]);
                    acc[j] = fmaf(__uint_as_float(word[i] & 0xffff0000u), xs[k + 2 * i + 1], acc[j]);
                }
            }
        }
    } else {
        for (int k = lane; k < K; k += 64) {
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] = fmaf(to_float(rows[j][k]), xs[k], acc[j]);
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) out[j] = wave_sum(acc[j]);
}

// A workgroup a row; its first wave chooses.  z [n, stride] are the router's 32-bit logits over `total` outputs.
// s = softmax(z); the choice goes
// by s + correction; outputs form `groups` equal groups of neighbours, a group counts by its largest choice score and
// only members of the `kept` best groups can be chosen (the others count as minus infinity); the `top` largest are
// chosen (the lower index among equals), in that order; a chosen output weighs s, divided, with `normalised`, by the
// chosen ones' sum plus weight_eps.  Rows at position -1 choose nothing (-1, weight 0).
// With `x` [n, W] and the router's matrix `w` [total, W] (both of type T) the workgroup works the logits out itself
// first, all its waves at it, 32-bit sums of the products in an order that W alone fixes: for steps of few rows, where
// a product's launch costs more than the product.  (The waves behind the first then walk through the choice with
// nothing to do, so that every barrier is met by all.)
template <typename T>
__global__ __launch_bounds__(256) void router_select_kernel(const float* __restrict__ z, int stride, const float* __restrict__ correction,
                                                            const int* __restrict__ positions, int total_all, int top, int groups_all,
                                                            int kept, int normalised, float weight_eps, int* __restrict__ choice,
                                                            float* __restrict__ weight, const T* __restrict__ x,
                                                            const T* __restrict__ w, int W) {
    extern __shared__ float router_lds[];             // score [total], choice score [total], group score [groups], kept or not [groups]
    float* score = router_lds;                        // (and behind them, where the logits are worked out here: logits [total], the row [W])
    float* pick = router_lds + total_all;
    float* group = pick + total_all;
    float* stays = group + groups_all;
    const int t = blockIdx.x, lane = threadIdx.x % PL_WAVE, wave = threadIdx.x / PL_WAVE, waves = blockDim.x / PL_WAVE;
    const bool chooser = wave == 0;
    int* chosen = choice + static_cast<size_t>(t) * top;
    float* counts = weight + static_cast<size_t>(t) * top;
    if (positions != nullptr && positions[t] < 0) {
        for (int c = threadIdx.x; c < top; c += blockDim.x) {
            chosen[c] = -1;
            counts[c] = 0.f;
        }
        return;
    }
    const float* row = z + static_cast<size_t>(t) * stride;
    if (x != nullptr) {
        float* logits = stays + groups_all;
        float* xs = logits + total_all;
        for (int k = threadIdx.x; k < W; k += blockDim.x) xs[k] = to_float(x[static_cast<size_t>(t) * W + k]);
        __syncthreads();
        for (int e0 = wave; e0 < total_all; e0 += 4 * waves) {
            float sums[4];
            router_dots<T>(w, xs, W, lane, e0, waves, total_all, sums);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (lane == 0 && e0 + j * waves < total_all) logits[e0 + j * waves] = sums[j];
        }
        __syncthreads();
        row = logits;
    }
    // (a wave that does not choose sees no outputs and no groups)
    const int total = chooser ? total_all : 0, groups = chooser ? groups_all : 0;
    float largest = -INFINITY;
    for (int e = lane; e < total; e += PL_WAVE) largest = fmaxf(largest, row[e]);
    largest = wave_max(largest);
    float sum = 0.f;
    for (int e = lane; e < total; e += PL_WAVE) {
        const float v = expf(row[e] - largest);
        score[e] = v;
        sum += v;
    }
    sum = wave_sum(sum);
    for (int e = lane; e < total; e += PL_WAVE) {
        const float s = score[e] / sum;
        score[e] = s;
        pick[e] = correction != nullptr ? s + correction[e] : s;
    }
    __syncthreads();
    if (groups_all > 1) {
        const int size = total_all / groups_all;
        for (int g = lane; g < groups; g += PL_WAVE) {
            float best = -INFINITY;
            for (int e = g * size; e < (g + 1) * size; ++e) best = fmaxf(best, pick[e]);
            group[g] = best;
            stays[g] = 0.f;
        }
        __syncthreads();
        // the best `kept` groups keep their members, the others' members leave
        for (int k = 0; k < kept; ++k) {
            float v = -INFINITY;
            int at = 0x7fffffff;
            for (int g = lane; g < groups; g += PL_WAVE) {
                const float s = group[g];
                if (stays[g] == 0.f && (at == 0x7fffffff || s > v)) {
                    v = s;
                    at = g;
                }
            }
            wave_best(v, at);
            if (chooser && lane == 0 && at != 0x7fffffff) stays[at] = 1.f;
            __syncthreads();
        }
        for (int e = lane; e < total; e += PL_WAVE)
            if (stays[e / size] == 0.f) pick[e] = -INFINITY;
        __syncthreads();
    }
    float chosen_sum = 0.f;
    for (int c = 0; c < top; ++c) {
        float v = -INFINITY;
        int at = 0x7fffffff;
        for (int e = lane; e < total; e += PL_WAVE) {
            const float s = pick[e];
            if (!isnan(s) && (s > v || (s == v && e < at))) {
                v = s;
                at = e;
            }
        }
        wave_best(v, at);
        if (at == 0x7fffffff) at = -1;               // (nothing left to choose from)
        const float s = (chooser && at >= 0) ? score[at] : 0.f;
        chosen_sum += s;
        if (chooser && lane == 0) {
            chosen[c] = at;
            counts[c] = s;
            if (at >= 0) pick[at] = NAN;             // (taken: below every other value, minus infinity included)
        }
        __syncthreads();
    }
    if (normalised && chooser) {
        for (int c = lane; c < top; c += PL_WAVE) counts[c] = counts[c] / (chosen_sum + weight_eps);
    }
}

// z [n, stride] holds the logits, or, where it is null, x [n, W] and w [total, W] of type `dtype` give them.
extern "C" int pl_router_select(const float* z, int stride, const float* correction, const int* positions, int n, int total,
                                int top, int groups, int kept, int normalised, float weight_eps, int* choice, float* weight,
                                const void* x, const void* w, int W, int dtype, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && total > 0 && total <= 8192 && top > 0 && top <= total && (z == nullptr || stride >= total),
               "router_select: %d rows, %d of %d outputs in rows of %d", n, top, total, stride);
    PL_REQUIRE((z != nullptr) != (x != nullptr) && (x == nullptr || (w != nullptr && W > 0 && W <= 8192 && total <= 1024)),
               "router_select: logits, or rows of up to 8192 and a router of up to 1024 outputs to work them out from");
    PL_REQUIRE(groups >= 1 && total % groups == 0 && kept >= 1 && kept <= groups && top <= kept * (total / groups),
               "router_select: %d outputs in %d groups of which %d are kept, %d chosen", total, groups, kept, top);
    if (n == 0) return 0;
    size_t lds = 2 * (static_cast<size_t>(total) + groups) * sizeof(float);
    if (x == nullptr) {
        router_select_kernel<float><<<n, 64, lds, stream>>>(z, stride, correction, positions, total, top, groups, kept, normalised,
                                                            weight_eps, choice, weight, nullptr, nullptr, 0);
    } else {
        lds += (static_cast<size_t>(total) + W) * sizeof(float);
        if (dtype == PL_DTYPE_F32)
            router_select_kernel<float><<<n, 256, lds, stream>>>(nullptr, 0, correction, positions, total, top, groups, kept, normalised,
                                                                weight_eps, choice, weight, static_cast<const float*>(x),
                                                                static_cast<const float*>(w), W);
        else if (dtype == PL_DTYPE_BF16)
            router_select_kernel<bf16_t><<<n, 256, lds, stream>>>(nullptr, 0, correction, positions, total, top, groups, kept, normalised,
                                                                 weight_eps, choice, weight, static_cast<const bf16_t*>(x),
                                                                 static_cast<const bf16_t*>(w), W);
        else
            PL_REQUIRE(false, "router_select: dtype code %d", dtype);
    }
    PL_CHECK_LAUNCH("router_select");
    return 0;
}
