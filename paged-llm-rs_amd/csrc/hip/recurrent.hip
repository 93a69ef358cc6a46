// Mixers that carry a matrix of state from token to token instead of keys and values in pages:
// linear attention with a fixed decay a head, the matrix memory with exponential gates, and the gated
// delta rule; the short causal convolution with its carried history; and the norm over groups of the
// read-out, multiplied by a gate.  States, gates, decays and read-outs are 32-bit whatever the model's
// type is; the rows these kernels read are the 32-bit sums of the projections.
//
// A request's tokens of the step are rows q_start[s] .. q_start[s] + q_len[s] - 1; its state lives in
// slot state_slots[s] of a [slots, floats a slot] tensor.  A request without a slot (padding) is skipped.
#include "recurrent.hpp"

#define PL_SCAN_CHUNK 16      // tokens staged in LDS at a time

// The rows i of a lane's column of S, in blocks of 16 (a block that starts behind D is skipped).
#define PL_ROWS_OF_S                                  \
    _Pragma("unroll") for (int ib = 0; ib < DMAX; ib += 16) \
        if (ib < D)                                   \
            _Pragma("unroll") for (int i = ib; i < ib + 16; ++i)

// One wave owns 64 columns of one head's S for one request and walks the request's tokens in order.
// Lane j holds column j of S (D values in registers), so S^T k and S^T q are sums inside a lane, taken
// in ascending row order: a token's result does not depend on how the tokens were cut into steps.
template <int KIND, int DMAX>
__global__ __launch_bounds__(64) void scan_kernel(ScanArgs a) {
    extern __shared__ float lds[];
    const int lane = threadIdx.x;
    const int h = blockIdx.y, s = blockIdx.z;
    const int slot = a.state_slots[s];
    const int n = a.q_len[s];
    if (slot < 0 || n <= 0 || (a.below > 0 && n >= a.below)) return;
    const int start = a.q_start[s];
    const int D = a.D, V = a.V, H = a.H;
    const int g = h / (H / a.G);
    const int j = blockIdx.x * 64 + lane;
    const bool owns = j < V;

    // q and k are staged in rows of Dp = D rounded up to 16, zeros behind D: the rows of S behind D then
    // stay zero, and the loops over S run in whole blocks of 16 rows
    const int Dp = (D + 15) & ~15;
    float* qs = lds;                              // [CHUNK][Dp]
    float* ks = qs + PL_SCAN_CHUNK * Dp;          // [CHUNK][Dp]
    float* vs = ks + PL_SCAN_CHUNK * Dp;          // [CHUNK][64]
    float* g1 = vs + PL_SCAN_CHUNK * 64;          // [CHUNK]
    float* g2 = g1 + PL_SCAN_CHUNK;               // [CHUNK]
    float* nrm = g2 + PL_SCAN_CHUNK;              // [2 * CHUNK]

    float* slot_state = a.state + static_cast<size_t>(slot) * a.state_stride;
    float* Sg = slot_state + a.s_off + static_cast<size_t>(h) * D * V;
    float S[DMAX];
#pragma unroll
    for (int i = 0; i < DMAX; ++i) S[i] = (owns && i < D) ? Sg[static_cast<size_t>(i) * V + j] : 0.f;

    // mlstm: the normaliser n is dealt over the lanes (lane l holds rows l, l + 64, ...), every wave of
    // a head keeps its own copy, and n . q is a sum over the wave in a fixed order.
    constexpr int NPER = (DMAX + 63) / 64;
    float nv[NPER];
    float m = 0.f;
    // (Every tile of columns has a copy of n and m of its own in the slot, n [H, tiles, D] and m [H, tiles]: a
    // tile that starts after another has finished must not read what that one wrote.)
    const int tiles = gridDim.x;
    if (KIND == PL_SCAN_MLSTM) {
        const float* ng = slot_state + a.n_off + (static_cast<size_t>(h) * tiles + blockIdx.x) * D;
#pragma unroll
        for (int r = 0; r < NPER; ++r) nv[r] = (lane + 64 * r < D) ? ng[lane + 64 * r] : 0.f;
        m = slot_state[a.m_off + h * tiles + blockIdx.x];
    }
    float decay = 0.f, a_rate = 0.f, dt_bias = 0.f, bias_i = 0.f, bias_f = 0.f;
    if (KIND == PL_SCAN_LIGHTNING) decay = a.p1[h];
    if (KIND == PL_SCAN_DELTA) { a_rate = expf(a.p1[h]); dt_bias = a.p2[h]; }
    if (KIND == PL_SCAN_MLSTM) { bias_i = a.p1[h]; bias_f = a.p2[h]; }
    const float q_scale = 1.f / sqrtf(static_cast<float>(D));
    const int HV = H * V;

    for (int c0 = 0; c0 < n; c0 += PL_SCAN_CHUNK) {
        const int count = min(PL_SCAN_CHUNK, n - c0);
        // ---- stage the chunk's q, k, v and gates ----
        for (int e = lane; e < count * Dp; e += 64) {
            const int t = e / Dp, i = e - t * Dp;
            float q = 0.f, k = 0.f;
            if (i < D) {
                const float* row = a.qkv + static_cast<size_t>(start + c0 + t) * a.qkv_stride;
                q = row[a.q_off + g * D + i];
                k = row[a.k_off + g * D + i];
                if (KIND == PL_SCAN_LIGHTNING) { q = silu_f(q); k = silu_f(k); }
                if (KIND == PL_SCAN_MLSTM) q *= q_scale;
            }
            qs[e] = q;
            ks[e] = k;
        }
        for (int e = lane; e < count * 64; e += 64) {
            const int t = e / 64;
            const float* row = a.qkv + static_cast<size_t>(start + c0 + t) * a.qkv_stride;
            float v = owns ? row[a.v_off + h * V + j] : 0.f;
            if (KIND == PL_SCAN_LIGHTNING) v = silu_f(v);
            vs[t * 64 + lane] = v;
        }
        if (KIND != PL_SCAN_LIGHTNING && lane < count) {
            const float* row = a.gates + static_cast<size_t>(start + c0 + lane) * a.gates_stride;
            const float x1 = row[a.g1_off + h], x2 = row[a.g2_off + h];
            if (KIND == PL_SCAN_MLSTM) {
                g1[lane] = a.cap * tanhf((x1 + bias_i) / a.cap);
                g2[lane] = logsigmoid_f(a.cap * tanhf((x2 + bias_f) / a.cap));
            } else {
                g1[lane] = sigmoid_f(x1);
                g2[lane] = expf(-a_rate * softplus_f(x2 + dt_bias));
            }
        }
        __syncthreads();
        if (KIND == PL_SCAN_DELTA) {
            // q and k as unit vectors (q also times D^-1/2): the sums of squares in ascending order
            if (lane < 2 * count) {
                const float* x = (lane < count ? qs : ks) + (lane < count ? lane : lane - count) * Dp;
                float ss = 0.f;
                for (int i = 0; i < D; ++i) ss += x[i] * x[i];
                nrm[lane] = 1.f / sqrtf(ss + 1e-6f) * (lane < count ? q_scale : 1.f);
            }
            __syncthreads();
            for (int e = lane; e < count * Dp; e += 64) {
                const int t = e / Dp;
                qs[e] *= nrm[t];
                ks[e] *= nrm[count + t];
            }
            __syncthreads();
        }
        // ---- the tokens of the chunk, in order ----
        for (int t = 0; t < count; ++t) {
            const float* q = qs + t * Dp;
            const float* k = ks + t * Dp;
            const float v = vs[t * 64 + lane];
            float o = 0.f;
            if (KIND == PL_SCAN_LIGHTNING) {
                PL_ROWS_OF_S {
                        S[i] = decay * S[i] + k[i] * v;
                        o += S[i] * q[i];
                    }
            } else if (KIND == PL_SCAN_MLSTM) {
                const float gi = g1[t], gf = g2[t];
                const float m_new = fmaxf(gf + m, gi);
                const float keep = expf(gf + m - m_new), add = expf(gi - m_new);
                m = m_new;
                float part = 0.f;
#pragma unroll
                for (int r = 0; r < NPER; ++r)
                    if (lane + 64 * r < D) {
                        nv[r] = keep * nv[r] + add * k[lane + 64 * r];
                        part += nv[r] * q[lane + 64 * r];
                    }
                const float nq = wave_sum(part);
                const float av = add * v;
                PL_ROWS_OF_S {
                        S[i] = keep * S[i] + k[i] * av;
                        o += S[i] * q[i];
                    }
                o = o / (fmaxf(fabsf(nq), expf(-m_new)) + 1e-6f);
            } else {
                const float beta = g1[t], gd = g2[t];
                float mem = 0.f;
                PL_ROWS_OF_S {
                        S[i] *= gd;
                        mem += S[i] * k[i];
                    }
                const float u = beta * (v - mem);
                PL_ROWS_OF_S {
                        S[i] += k[i] * u;
                        o += S[i] * q[i];
                    }
            }
            if (owns) a.out[static_cast<size_t>(start + c0 + t) * HV + h * V + j] = o;
        }
        __syncthreads();
    }
    if (owns) {
#pragma unroll
        for (int i = 0; i < DMAX; ++i)
            if (i < D) Sg[static_cast<size_t>(i) * V + j] = S[i];
    }
    if (KIND == PL_SCAN_MLSTM) {
        float* ng = slot_state + a.n_off + (static_cast<size_t>(h) * tiles + blockIdx.x) * D;
#pragma unroll
        for (int r = 0; r < NPER; ++r)
            if (lane + 64 * r < D) ng[lane + 64 * r] = nv[r];
        if (lane == 0) slot_state[a.m_off + h * tiles + blockIdx.x] = m;
    }
}

template <int KIND>
static int launch_scan(const ScanArgs& a, int seqs, hipStream_t stream) {
    const dim3 grid(pl_ceil_div(a.V, 64), a.H, seqs);
    const size_t lds = static_cast<size_t>(PL_SCAN_CHUNK) * (2 * ((a.D + 15) & ~15) + 64 + 4) * sizeof(float);
    if (a.D <= 16) scan_kernel<KIND, 16><<<grid, 64, lds, stream>>>(a);
    else if (a.D <= 32) scan_kernel<KIND, 32><<<grid, 64, lds, stream>>>(a);
    else if (a.D <= 64) scan_kernel<KIND, 64><<<grid, 64, lds, stream>>>(a);
    else if (a.D <= 128) scan_kernel<KIND, 128><<<grid, 64, lds, stream>>>(a);
    else scan_kernel<KIND, 256><<<grid, 64, lds, stream>>>(a);
    PL_CHECK_LAUNCH("recurrent_scan");
    return 0;
}

extern "C" int pl_recurrent_scan(int kind, const float* qkv, int qkv_stride, int q_off, int k_off, int v_off,
                                 const float* gates, int gates_stride, int g1_off, int g2_off,
                                 const float* p1, const float* p2, float cap,
                                 float* state, long state_stride, int s_off, int n_off, int m_off,
                                 float* out, const int* q_start, const int* q_len, const int* state_slots,
                                 int seqs, int H, int G, int D, int V, int below, hipStream_t stream) {
    PL_REQUIRE(kind >= 0 && kind <= 2, "recurrent_scan: kind %d", kind);
    PL_REQUIRE(H > 0 && G > 0 && H % G == 0, "recurrent_scan: %d heads over %d heads of q and k", H, G);
    PL_REQUIRE(D > 0 && D <= 256 && V > 0, "recurrent_scan: a state of %d by %d a head (q and k up to 256)", D, V);
    PL_REQUIRE(seqs >= 0 && seqs <= 65535 && H <= 65535, "recurrent_scan: %d requests, %d heads", seqs, H);
    PL_REQUIRE(kind == PL_SCAN_LIGHTNING || (gates != nullptr && p1 != nullptr && p2 != nullptr),
               "recurrent_scan: the gates of kind %d are missing", kind);
    PL_REQUIRE(kind != PL_SCAN_LIGHTNING || p1 != nullptr, "recurrent_scan: the decays are missing");
    PL_REQUIRE(kind != PL_SCAN_MLSTM || cap > 0.f, "recurrent_scan: a gate cap of %g", cap);
    if (seqs == 0) return 0;
    ScanArgs a{qkv, qkv_stride, q_off, k_off, v_off, gates, gates_stride, g1_off, g2_off, p1, p2, cap,
               state, state_stride, s_off, n_off, m_off, out, q_start, q_len, state_slots, H, G, D, V, below};
    if (kind == PL_SCAN_LIGHTNING) return launch_scan<PL_SCAN_LIGHTNING>(a, seqs, stream);
    if (kind == PL_SCAN_MLSTM) return launch_scan<PL_SCAN_MLSTM>(a, seqs, stream);
    return launch_scan<PL_SCAN_DELTA>(a, seqs, stream);
}

// ---------------------------------------------------------------------------
// Short causal convolution over time, a filter a channel:
//   y[t, c] = sum_j w[j, c] * u[t - taps + 1 + j, c]      (w is stored a tap a row)
// u are the columns [off, off + C) of the rows; the taps - 1 rows before a request's first row of the
// step come from its history hist[taps - 1][C] (zeros at a request's start), the last one the newest.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float conv_at(const float* __restrict__ rows, int stride, int off, int C,
                                         const float* __restrict__ w, int taps, const float* __restrict__ hist,
                                         int row, int r, int c) {
    float acc = 0.f;
    for (int jt = 0; jt < taps; ++jt) {
        const int back = taps - 1 - jt;
        const int src = r - back;
        const float u = src >= 0 ? rows[static_cast<size_t>(row - back) * stride + off + c]
                                 : hist[static_cast<size_t>(taps - 1 + src) * C + c];
        acc += w[jt * C + c] * u;
    }
    return acc;
}

__global__ void short_conv_kernel(const float* __restrict__ rows, int stride, int off, int C,
                                  const float* __restrict__ w, int taps, const float* __restrict__ state,
                                  long state_stride, int hist_off, const int* __restrict__ positions,
                                  const int* __restrict__ seq_of, const int* __restrict__ q_start,
                                  const int* __restrict__ state_slots, float* __restrict__ out, int act) {
    const int t = blockIdx.x;
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= C || positions[t] < 0) return;
    const int s = seq_of[t];
    const int slot = state_slots[s];
    if (slot < 0) return;
    const float* hist = state + static_cast<size_t>(slot) * state_stride + hist_off;
    const float y = conv_at(rows, stride, off, C, w, taps, hist, t, t - q_start[s], c);
    out[static_cast<size_t>(t) * C + c] = act ? silu_f(y) : y;
}

extern "C" int pl_short_conv(const float* rows, int stride, int off, int C, const float* w, int taps,
                             const float* state, long state_stride, int hist_off, const int* positions,
                             const int* seq_of, const int* q_start, const int* state_slots, float* out, int act,
                             int n, hipStream_t stream) {
    PL_REQUIRE(C > 0 && taps >= 1 && taps <= 16 && n >= 0, "short_conv: %d channels, %d taps, %d rows", C, taps, n);
    if (n == 0) return 0;
    short_conv_kernel<<<dim3(n, pl_ceil_div(C, 256)), 256, 0, stream>>>(rows, stride, off, C, w, taps, state, state_stride,
                                                                      hist_off, positions, seq_of, q_start, state_slots, out, act);
    PL_CHECK_LAUNCH("short_conv");
    return 0;
}

// After the convolution has read it: the history becomes the last taps - 1 inputs of each request, from
// the step's rows and, where the request brought fewer, from what the history held.
__global__ void conv_history_kernel(const float* __restrict__ rows, int stride, int off, int C, int taps,
                                    float* __restrict__ state, long state_stride, int hist_off,
                                    const int* __restrict__ q_start, const int* __restrict__ q_len,
                                    const int* __restrict__ state_slots) {
    const int s = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const int slot = state_slots[s];
    const int n = q_len[s];
    if (c >= C || slot < 0 || n <= 0) return;
    float* hist = state + static_cast<size_t>(slot) * state_stride + hist_off;
    const int start = q_start[s];
    float kept[16];
    for (int i = 0; i < taps - 1; ++i) {
        const int r = n - (taps - 1) + i;
        kept[i] = r >= 0 ? rows[static_cast<size_t>(start + r) * stride + off + c]
                         : hist[static_cast<size_t>(taps - 1 + r) * C + c];
    }
    for (int i = 0; i < taps - 1; ++i) hist[static_cast<size_t>(i) * C + c] = kept[i];
}

extern "C" int pl_conv_history(const float* rows, int stride, int off, int C, int taps, float* state,
                               long state_stride, int hist_off, const int* q_start, const int* q_len,
                               const int* state_slots, int seqs, hipStream_t stream) {
    PL_REQUIRE(C > 0 && taps >= 1 && taps <= 16 && seqs >= 0 && seqs <= 65535, "conv_history: %d channels, %d taps, %d requests", C, taps, seqs);
    if (seqs == 0 || taps == 1) return 0;
    conv_history_kernel<<<dim3(pl_ceil_div(C, 256), seqs), 256, 0, stream>>>(rows, stride, off, C, taps, state, state_stride,
                                                                           hist_off, q_start, q_len, state_slots);
    PL_CHECK_LAUNCH("conv_history");
    return 0;
}

// ---------------------------------------------------------------------------
// out[t, c] = x[t, c] / sqrt(mean over c's group of x^2 + eps) * gain[c mod gain_len] * act(gate[t, c])
// Groups are runs of `group` columns (a head, or the whole row).  One wave a row and group.
// act: 0 sigmoid, 1 silu, -1 no gate.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(64) void gated_group_norm_kernel(const float* __restrict__ x, int width, int group,
                                                              const float* __restrict__ gain, int gain_len, float eps,
                                                              const float* __restrict__ gate, int gate_stride,
                                                              int gate_off, int act, T* __restrict__ out) {
    const int t = blockIdx.x, first = blockIdx.y * group;
    const float* row = x + static_cast<size_t>(t) * width + first;
    // a lane keeps up to eight of its values between the sum and the output (groups up to 512 are read once)
    constexpr int KEEP = 8;
    float kept[KEEP];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
        const int e = threadIdx.x + 64 * k;
        kept[k] = e < group ? row[e] : 0.f;
        ss += kept[k] * kept[k];
    }
    for (int e = threadIdx.x + 64 * KEEP; e < group; e += 64) ss += row[e] * row[e];
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / static_cast<float>(group) + eps);
    const float* g = gate != nullptr ? gate + static_cast<size_t>(t) * gate_stride + gate_off + first : nullptr;
    T* o = out + static_cast<size_t>(t) * width + first;
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
        const int e = threadIdx.x + 64 * k;
        if (e < group) {
            float y = kept[k] * inv * gain[(first + e) % gain_len];
            if (act >= 0) y *= act == 0 ? sigmoid_f(g[e]) : silu_f(g[e]);
            o[e] = from_float<T>(y);
        }
    }
    for (int e = threadIdx.x + 64 * KEEP; e < group; e += 64) {
        float y = row[e] * inv * gain[(first + e) % gain_len];
        if (act >= 0) y *= act == 0 ? sigmoid_f(g[e]) : silu_f(g[e]);
        o[e] = from_float<T>(y);
    }
}

// The same for groups of more than 512 columns (all heads normalised together): a workgroup of four waves a row and
// group, so that a group of up to 2,048 is read once, every load asked for at once.
template <typename T>
__global__ __launch_bounds__(256) void gated_group_norm_wide_kernel(const float* __restrict__ x, int width, int group,
                                                                    const float* __restrict__ gain, int gain_len, float eps,
                                                                    const float* __restrict__ gate, int gate_stride,
                                                                    int gate_off, int act, T* __restrict__ out) {
    __shared__ float scratch[16];
    const int t = blockIdx.x, first = blockIdx.y * group;
    const float* row = x + static_cast<size_t>(t) * width + first;
    const float* g = gate != nullptr ? gate + static_cast<size_t>(t) * gate_stride + gate_off + first : nullptr;
    const float* gains = gain + (gain_len == width ? first : 0);     // (gain_len is the row's width or the group's)
    constexpr int KEEP = 8;
    float kept[KEEP], gates[KEEP], scale[KEEP];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
        const int e = threadIdx.x + 256 * k;
        kept[k] = e < group ? row[e] : 0.f;
        gates[k] = (e < group && act >= 0) ? g[e] : 0.f;
        scale[k] = e < group ? gains[e] : 0.f;
        ss += kept[k] * kept[k];
    }
    for (int e = threadIdx.x + 256 * KEEP; e < group; e += 256) ss += row[e] * row[e];
    ss = block_sum(ss, scratch);
    const float inv = 1.f / sqrtf(ss / static_cast<float>(group) + eps);
    T* o = out + static_cast<size_t>(t) * width + first;
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
        const int e = threadIdx.x + 256 * k;
        if (e < group) {
            float y = kept[k] * inv * scale[k];
            if (act >= 0) y *= act == 0 ? sigmoid_f(gates[k]) : silu_f(gates[k]);
            o[e] = from_float<T>(y);
        }
    }
    for (int e = threadIdx.x + 256 * KEEP; e < group; e += 256) {
        float y = row[e] * inv * gains[e];
        if (act >= 0) y *= act == 0 ? sigmoid_f(g[e]) : silu_f(g[e]);
        o[e] = from_float<T>(y);
    }
}

extern "C" int pl_gated_group_norm(const float* x, int n, int width, int group, const float* gain, int gain_len,
                                   float eps, const float* gate, int gate_stride, int gate_off, int act, void* out,
                                   int dtype, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && width > 0 && group > 0 && width % group == 0, "gated_group_norm: rows %d, width %d, groups of %d", n, width, group);
    PL_REQUIRE(gain_len > 0 && width % gain_len == 0 && (gain_len == width || gain_len == group),
               "gated_group_norm: %d gains for rows of %d in groups of %d", gain_len, width, group);
    PL_REQUIRE(act < 0 || gate != nullptr, "gated_group_norm: no gate");
    if (n == 0) return 0;
    PL_REQUIRE(width / group <= 65535, "gated_group_norm: %d groups a row", width / group);
    const dim3 grid(n, width / group);
    if (group > 512 && (dtype == PL_DTYPE_F32 || dtype == PL_DTYPE_BF16)) {
        if (dtype == PL_DTYPE_F32)
            gated_group_norm_wide_kernel<float><<<grid, 256, 0, stream>>>(x, width, group, gain, gain_len, eps, gate, gate_stride, gate_off, act, static_cast<float*>(out));
        else
            gated_group_norm_wide_kernel<bf16_t><<<grid, 256, 0, stream>>>(x, width, group, gain, gain_len, eps, gate, gate_stride, gate_off, act, static_cast<bf16_t*>(out));
        PL_CHECK_LAUNCH("gated_group_norm");
        return 0;
    }
    if (dtype == PL_DTYPE_F32)
        gated_group_norm_kernel<float><<<grid, 64, 0, stream>>>(x, width, group, gain, gain_len, eps, gate, gate_stride, gate_off, act, static_cast<float*>(out));
    else if (dtype == PL_DTYPE_BF16)
        gated_group_norm_kernel<bf16_t><<<grid, 64, 0, stream>>>(x, width, group, gain, gain_len, eps, gate, gate_stride, gate_off, act, static_cast<bf16_t*>(out));
    else
        PL_REQUIRE(false, "gated_group_norm: dtype code %d", dtype);
    PL_CHECK_LAUNCH("gated_group_norm");
    return 0;
}
