// What attention layers without a gain on q and k do between their projections and the attention kernels.
//
// head_prepare: for every token and head of a projected row [q | k | v] (32-bit sums, plus the projections' biases
// where they have any): q and k divided by
// their root mean square over the head (optional, with an optional gain), the rotation of a stretch of the
// head (optional: value 2i with value 2i + 1, from tables of cosines and sines), q times a temperature that
// grows with the logarithm of the position (optional), then q into the query buffer and k and v into the
// request's pages.  Heads are stored in rows of Dp values with zeros behind a head's own size, so that query,
// key and value heads of different sizes share the attention kernels' one head size.
//
// latent_prepare: the same place in a layer whose pages hold one small vector a token: of a projected row
// [q | ... | small vector, rotated key part] the small vector is normalised (gain), the key part rotated, and
// both go into the token's row of the pages, [vector | key part | zeros]; a query head's unrotated part is
// stored head-major for the product that carries it into the small vector's space, and its rotated part goes
// behind the place that product fills in the query row, [kv_rank to be filled | rotated part | zeros].
//
// Statistics, angles, temperatures and rotations are 32-bit; a value is rounded once, when it is stored.
#include "common.hpp"

struct HeadPrepareArgs {
    const float* rows;        // [n, stride]: q | k | v from column `off`
    const float* bias;        // [H D + G D + G V] added to q | k | v first, or null
    int stride, off;
    int unit;                 // q and k divided by their root mean square
    float eps;
    const float* q_gain;      // [D] or null
    const float* k_gain;
    const float* cos;         // [positions, rot / 2] or null
    const float* sin;
    int rot_off, rot, table_rows;
    int tempered;             // q times 1 + coef * ln(floor((p + 1) / every) + 1)
    float temp_coef;
    int temp_every;
    const int* positions;
    const int* seq_of;
    const int* block_table;
    int max_blocks, block_size, write_kv;
    void* q_out;              // [n, H * Dp]
    void* k_pool;             // [pages * block_size, G * Dp]
    void* v_pool;
    int H, G, D, V, Dp;
};

// A wave a token and head (a query head, a key head or a value head).
template <typename T>
__global__ __launch_bounds__(64) void head_prepare_kernel(HeadPrepareArgs a) {
    __shared__ float head[1024];
    const int t = blockIdx.x, which = blockIdx.y, lane = threadIdx.x;
    const int pos = a.positions[t];
    if (pos < 0) return;
    const int H = a.H, G = a.G, D = a.D, V = a.V, Dp = a.Dp;
    const int kind = which < H ? 0 : (which < H + G ? 1 : 2);
    if (kind != 0 && !a.write_kv) return;
    const int index = kind == 0 ? which : (kind == 1 ? which - H : which - H - G);
    const int width = kind == 2 ? V : D;
    const int c0 = kind == 0 ? index * D : (kind == 1 ? H * D + index * D : H * D + G * D + index * V);
    const float* src = a.rows + static_cast<size_t>(t) * a.stride + a.off + c0;
    const float* bias = a.bias != nullptr ? a.bias + c0 : nullptr;

    float ss = 0.f;
    for (int e = lane; e < width; e += 64) {
        const float x = bias != nullptr ? src[e] + bias[e] : src[e];
        head[e] = x;
        ss += x * x;
    }
    float mult = 1.f;
    if (kind != 2 && a.unit) {
        ss = wave_sum(ss);
        mult = 1.f / sqrtf(ss / static_cast<float>(D) + a.eps);
    }
    const float* gain = kind == 0 ? a.q_gain : (kind == 1 ? a.k_gain : nullptr);
    if (kind != 2) {
        for (int e = lane; e < width; e += 64) head[e] = head[e] * mult * (gain != nullptr ? gain[e] : 1.f);
    }
    __syncthreads();
    float temper = 1.f;
    if (kind == 0 && a.tempered)
        temper = 1.f + a.temp_coef * logf(static_cast<float>((pos + 1) / a.temp_every + 1));

    T* dst;
    if (kind == 0) {
        dst = static_cast<T*>(a.q_out) + (static_cast<size_t>(t) * H + index) * Dp;
    } else {
        const int s = a.seq_of[t];
        const int page = a.block_table[static_cast<size_t>(s) * a.max_blocks + pos / a.block_size];
        if (page < 0) return;
        const size_t row = static_cast<size_t>(page) * a.block_size + pos % a.block_size;
        dst = static_cast<T*>(kind == 1 ? a.k_pool : a.v_pool) + (row * G + index) * Dp;
    }
    const bool turns = kind != 2 && a.rot > 0 && pos < a.table_rows;
    const float* cs = a.cos + static_cast<size_t>(turns ? pos : 0) * (a.rot / 2);
    const float* sn = a.sin + static_cast<size_t>(turns ? pos : 0) * (a.rot / 2);
    for (int e = lane; e < Dp; e += 64) {
        float x = 0.f;
        if (e < width) {
            x = head[e];
            const int r = e - a.rot_off;
            if (turns && r >= 0 && r < a.rot) {
                const int i = r >> 1;
                x = (r & 1) ? head[e] * cs[i] + head[e - 1] * sn[i] : head[e] * cs[i] - head[e + 1] * sn[i];
            }
            x *= temper;
        }
        dst[e] = from_float<T>(x);
    }
}

extern "C" int pl_head_prepare(const float* rows, const float* bias, int stride, int off, int unit, float eps, const float* q_gain,
                               const float* k_gain, const float* cos, const float* sin, int rot_off, int rot,
                               int table_rows, int tempered, float temp_coef, int temp_every, const int* positions,
                               const int* seq_of, const int* block_table, int max_blocks, int block_size, int write_kv,
                               void* q_out, void* k_pool, void* v_pool, int dtype, int n, int H, int G, int D, int V,
                               int Dp, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && H > 0 && G > 0 && H % G == 0 && H + 2 * G <= 65535, "head_prepare: rows %d, %d query heads over %d key heads", n, H, G);
    PL_REQUIRE(D > 0 && V > 0 && Dp >= D && Dp >= V && Dp <= 1024, "head_prepare: heads of %d and %d in rows of %d (up to 1024)", D, V, Dp);
    PL_REQUIRE(rot >= 0 && rot % 2 == 0 && rot_off >= 0 && rot_off + rot <= D && (rot == 0 || (cos != nullptr && sin != nullptr && table_rows > 0)),
               "head_prepare: a rotation over %d values from %d on of a head of %d", rot, rot_off, D);
    PL_REQUIRE(block_size > 0 && max_blocks > 0 && (!tempered || temp_every > 0), "head_prepare: pages of %d, tables of %d, a temperature every %d", block_size, max_blocks, temp_every);
    PL_REQUIRE(stride >= off + H * D + G * D + G * V, "head_prepare: rows of %d values for %d + %d + %d from %d on", stride, H * D, G * D, G * V, off);
    if (n == 0) return 0;
    HeadPrepareArgs a{rows, bias, stride, off, unit, eps, q_gain, k_gain, cos, sin, rot_off, rot, table_rows, tempered, temp_coef,
                      temp_every, positions, seq_of, block_table, max_blocks, block_size, write_kv, q_out, k_pool, v_pool,
                      H, G, D, V, Dp};
    const dim3 grid(n, H + 2 * G);
    if (dtype == PL_DTYPE_F32) head_prepare_kernel<float><<<grid, 64, 0, stream>>>(a);
    else if (dtype == PL_DTYPE_BF16) head_prepare_kernel<bf16_t><<<grid, 64, 0, stream>>>(a);
    else PL_REQUIRE(false, "head_prepare: dtype code %d", dtype);
    PL_CHECK_LAUNCH("head_prepare");
    return 0;
}

// ---- q and k normed over all their heads at once, values that are the keys as projected ------------------------

struct WidePrepareArgs {
    const float* rows;        // [n, stride]: q | k from column `off`
    const float* bias;        // [H D + G D] added to q | k first, or null
    int stride, off;
    int normed;               // q divided by its root mean square over all H D values, k over all G D
    float eps;
    const float* q_gain;      // [H D] or null
    const float* k_gain;      // [G D] or null
    const float* freq;        // [rot / 2]: the angle of pair i is position * freq[i], in 32-bit
    int rot;                  // the first `rot` values of every head turn in pairs (2i, 2i + 1)
    const int* positions;
    const int* seq_of;
    const int* block_table;
    int max_blocks, block_size, write_kv;
    void* q_out;              // [n, H * Dp]
    void* k_pool;             // [pages * block_size, G * Dp]: the keys, normed and turned
    void* v_pool;             // the same shape: the keys as projected (bias included)
    int H, G, D, Dp;
};

// A workgroup a token.  The row of q | k (with the biases) waits in LDS, each value times its gain (and the keys a
// second time as they are: they are the values); two sums of squares over the whole projections; then a wave takes
// a head at a time: normed, turned and stored, heads in rows of Dp values with zeros behind.  Every load from memory
// stands before the first store, so none of them waits for one.
template <typename T>
__global__ __launch_bounds__(256) void wide_prepare_kernel(WidePrepareArgs a) {
    extern __shared__ float wide_lds[];               // [H D + G D] gained values, [G D] keys as projected, cosines, sines
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const int pos = a.positions[t];
    if (pos < 0) return;
    const int H = a.H, G = a.G, D = a.D, Dp = a.Dp, half = a.rot / 2;
    const int nq = H * D, nk = a.write_kv ? G * D : 0;
    float* gained = wide_lds;
    float* raw = wide_lds + (H + G) * D;
    float* cs = raw + G * D;
    float* sn = cs + half;
    const float* src = a.rows + static_cast<size_t>(t) * a.stride + a.off;
    float ssq = 0.f, ssk = 0.f;
    if ((a.stride | a.off | nq | nk) % 4 == 0) {
        for (int e = threadIdx.x * 4; e < nq + nk; e += blockDim.x * 4) {
            float4 x = *reinterpret_cast<const float4*>(src + e);
            if (a.bias != nullptr) {
                const float4 b = *reinterpret_cast<const float4*>(a.bias + e);
                x.x += b.x, x.y += b.y, x.z += b.z, x.w += b.w;
            }
            const float* gain = e < nq ? a.q_gain : a.k_gain;
            float4 g = {1.f, 1.f, 1.f, 1.f};
            if (gain != nullptr) g = *reinterpret_cast<const float4*>(gain + (e < nq ? e : e - nq));
            const float ss = x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
            if (e < nq) {
                ssq += ss;
            } else {
                ssk += ss;
                *reinterpret_cast<float4*>(raw + e - nq) = x;
            }
            *reinterpret_cast<float4*>(gained + e) = make_float4(x.x * g.x, x.y * g.y, x.z * g.z, x.w * g.w);
        }
    } else {
        for (int e = threadIdx.x; e < nq + nk; e += blockDim.x) {
            const float x = a.bias != nullptr ? src[e] + a.bias[e] : src[e];
            const float* gain = e < nq ? a.q_gain : a.k_gain;
            const float g = gain != nullptr ? gain[e < nq ? e : e - nq] : 1.f;
            if (e < nq) {
                ssq += x * x;
            } else {
                ssk += x * x;
                raw[e - nq] = x;
            }
            gained[e] = x * g;
        }
    }
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        float s_i, c_i;
        sincosf(static_cast<float>(pos) * a.freq[i], &s_i, &c_i);
        cs[i] = c_i;
        sn[i] = s_i;
    }
    T* k_dst = nullptr;
    T* v_dst = nullptr;
    if (nk > 0) {
        const int s = a.seq_of[t];
        const int page = a.block_table[static_cast<size_t>(s) * a.max_blocks + pos / a.block_size];
        if (page >= 0) {
            const size_t row = static_cast<size_t>(page) * a.block_size + pos % a.block_size;
            k_dst = static_cast<T*>(a.k_pool) + row * G * Dp;
            v_dst = static_cast<T*>(a.v_pool) + row * G * Dp;
        }
    }
    float inv_q = 1.f, inv_k = 1.f;
    if (a.normed) {
        ssq = block_sum(ssq, scratch);
        inv_q = 1.f / sqrtf(ssq / static_cast<float>(nq) + a.eps);
        if (nk > 0) {
            ssk = block_sum(ssk, scratch);
            inv_k = 1.f / sqrtf(ssk / static_cast<float>(nk) + a.eps);
        }
    }
    __syncthreads();
    T* q_dst = static_cast<T*>(a.q_out) + static_cast<size_t>(t) * H * Dp;
    const int lane = threadIdx.x % PL_WAVE, wave = threadIdx.x / PL_WAVE, waves = blockDim.x / PL_WAVE;
    const int heads = H + (k_dst != nullptr ? G : 0);
    for (int head = wave; head < heads; head += waves) {
        const bool query = head < H;
        const float inv = query ? inv_q : inv_k;
        const float* mine = gained + head * D;                            // (the keys' heads follow the queries')
        T* dst = query ? q_dst + head * Dp : k_dst + (head - H) * Dp;
        for (int d = lane; d < Dp; d += PL_WAVE) {
            float x = 0.f;
            if (d < D) {
                x = mine[d] * inv;
                if (d < a.rot) {
                    const float y = mine[(d & 1) ? d - 1 : d + 1] * inv;
                    const int i = d >> 1;
                    x = (d & 1) ? x * cs[i] + y * sn[i] : x * cs[i] - y * sn[i];
                }
            }
            dst[d] = from_float<T>(x);
            if (!query) v_dst[(head - H) * Dp + d] = from_float<T>(d < D ? raw[(head - H) * D + d] : 0.f);
        }
    }
}

extern "C" int pl_wide_prepare(const float* rows, const float* bias, int stride, int off, int normed, float eps,
                               const float* q_gain, const float* k_gain, const float* freq, int rot, const int* positions,
                               const int* seq_of, const int* block_table, int max_blocks, int block_size, int write_kv,
                               void* q_out, void* k_pool, void* v_pool, int dtype, int n, int H, int G, int D, int Dp,
                               hipStream_t stream) {
    PL_REQUIRE(n >= 0 && H > 0 && G > 0 && H % G == 0, "wide_prepare: rows %d, %d query heads over %d key heads", n, H, G);
    PL_REQUIRE(D > 0 && Dp >= D && Dp <= 1024, "wide_prepare: heads of %d in rows of %d (up to 1024)", D, Dp);
    PL_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= D && (rot == 0 || freq != nullptr),
               "wide_prepare: a rotation over %d values of a head of %d", rot, D);
    PL_REQUIRE(block_size > 0 && max_blocks > 0 && stride >= off + (H + G) * D, "wide_prepare: pages of %d, tables of %d, rows of %d values for %d from %d on",
               block_size, max_blocks, stride, (H + G) * D, off);
    const size_t lds = (static_cast<size_t>(H + 2 * G) * D + rot) * sizeof(float);
    PL_REQUIRE(lds <= 160 * 1024 - 256, "wide_prepare: %d + %d heads of %d are more than a workgroup's LDS holds", H, G, D);
    PL_REQUIRE(dtype == PL_DTYPE_F32 || dtype == PL_DTYPE_BF16, "wide_prepare: dtype code %d", dtype);
    if (n == 0) return 0;
    WidePrepareArgs a{rows, bias, stride, off, normed, eps, q_gain, k_gain, freq, rot, positions, seq_of, block_table,
                      max_blocks, block_size, write_kv, q_out, k_pool, v_pool, H, G, D, Dp};
    if (lds > 48 * 1024) {
        // (a launch that asks for more than 48 KB says so first)
        const void* kernel = dtype == PL_DTYPE_F32 ? reinterpret_cast<const void*>(&wide_prepare_kernel<float>)
                                                   : reinterpret_cast<const void*>(&wide_prepare_kernel<bf16_t>);
        const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
        PL_REQUIRE(e == hipSuccess, "wide_prepare: %zu bytes of LDS: %s", lds, hipGetErrorString(e));
    }
    if (dtype == PL_DTYPE_F32) wide_prepare_kernel<float><<<n, 256, lds, stream>>>(a);
    else wide_prepare_kernel<bf16_t><<<n, 256, lds, stream>>>(a);
    PL_CHECK_LAUNCH("wide_prepare");
    return 0;
}

struct LatentPrepareArgs {
    const float* rows;        // [n, stride]
    int stride;
    int q_off;                // H heads of [D | rot] from here
    int kv_off;               // [R | rot] from here (unused when nothing is written)
    const float* gain;        // [R]
    float eps;
    const float* cos;         // [positions, turned / 2]
    const float* sin;
    int turned, table_rows;   // the first `turned` values of a rotated part turn
    const int* positions;
    const int* seq_of;
    const int* block_table;
    int max_blocks, block_size, write_kv;
    void* q_plain;            // [H, n, D]: the unrotated parts, head-major
    void* q_out;              // [n, H * P]; values R .. P - 1 of every head are written here
    void* pool;               // [pages * block_size, P]
    int n, H, D, rot, R, P;
};

// A wave a token and job: jobs 0 .. H - 1 are the query heads, job H is the token's row of the pages.
template <typename T>
__global__ __launch_bounds__(64) void latent_prepare_kernel(LatentPrepareArgs a) {
    const int t = blockIdx.x, job = blockIdx.y, lane = threadIdx.x;
    const int pos = a.positions[t];
    if (pos < 0) return;
    const int H = a.H, D = a.D, rot = a.rot, R = a.R, P = a.P;
    // (without tables, `cos` lists the frequencies and the angle is position * frequency, in 32-bit)
    const bool tables = a.sin != nullptr;
    const bool turns = a.turned > 0 && (!tables || pos < a.table_rows);
    const float* cs = a.cos + static_cast<size_t>(turns && tables ? pos : 0) * (a.turned / 2);
    const float* sn = tables ? a.sin + static_cast<size_t>(turns ? pos : 0) * (a.turned / 2) : nullptr;
    const float* row = a.rows + static_cast<size_t>(t) * a.stride;
    const float* part;        // the rotated part this job turns
    T* dst;                   // where it goes, with the zeros behind it
    if (job < H) {
        const float* src = row + a.q_off + static_cast<size_t>(job) * (D + rot);
        T* plain = static_cast<T*>(a.q_plain) + (static_cast<size_t>(job) * a.n + t) * D;
        for (int e = lane; e < D; e += 64) plain[e] = from_float<T>(src[e]);
        part = src + D;
        dst = static_cast<T*>(a.q_out) + (static_cast<size_t>(t) * H + job) * P + R;
    } else {
        if (!a.write_kv) return;
        const int s = a.seq_of[t];
        const int page = a.block_table[static_cast<size_t>(s) * a.max_blocks + pos / a.block_size];
        if (page < 0) return;
        const float* src = row + a.kv_off;
        T* out = static_cast<T*>(a.pool) + (static_cast<size_t>(page) * a.block_size + pos % a.block_size) * P;
        float ss = 0.f;
        for (int e = lane; e < R; e += 64) ss += src[e] * src[e];
        ss = wave_sum(ss);
        const float inv = 1.f / sqrtf(ss / static_cast<float>(R) + a.eps);
        for (int e = lane; e < R; e += 64) out[e] = from_float<T>(src[e] * inv * a.gain[e]);
        part = src + R;
        dst = out + R;
    }
    for (int e = lane; e < P - R; e += 64) {
        float x = 0.f;
        if (e < rot) {
            x = part[e];
            if (turns && e < a.turned) {
                const int i = e >> 1;
                float c, sn_i;
                if (tables) {
                    c = cs[i];
                    sn_i = sn[i];
                } else {
                    sincosf(static_cast<float>(pos) * cs[i], &sn_i, &c);
                }
                x = (e & 1) ? part[e] * c + part[e - 1] * sn_i : part[e] * c - part[e + 1] * sn_i;
            }
        }
        dst[e] = from_float<T>(x);
    }
}

extern "C" int pl_latent_prepare(const float* rows, int stride, int q_off, int kv_off, const float* gain, float eps,
                                 const float* cos, const float* sin, int turned, int table_rows, const int* positions,
                                 const int* seq_of, const int* block_table, int max_blocks, int block_size, int write_kv,
                                 void* q_plain, void* q_out, void* pool, int dtype, int n, int H, int D, int rot, int R,
                                 int P, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && H > 0 && H < 65535 && D > 0 && rot >= 0 && R > 0 && P >= R + rot,
               "latent_prepare: rows %d, %d heads of %d + %d, vectors of %d in rows of %d", n, H, D, rot, R, P);
    PL_REQUIRE(turned >= 0 && turned % 2 == 0 && turned <= rot && (turned == 0 || (cos != nullptr && (sin == nullptr || table_rows > 0))),
               "latent_prepare: a rotation over %d of %d values", turned, rot);
    PL_REQUIRE(block_size > 0 && max_blocks > 0 && stride >= q_off + H * (D + rot) && (!write_kv || (stride >= kv_off + R + rot && gain != nullptr && pool != nullptr)),
               "latent_prepare: pages of %d, tables of %d, rows of %d values", block_size, max_blocks, stride);
    if (n == 0) return 0;
    LatentPrepareArgs a{rows, stride, q_off, kv_off, gain, eps, cos, sin, turned, table_rows, positions, seq_of, block_table,
                        max_blocks, block_size, write_kv, q_plain, q_out, pool, n, H, D, rot, R, P};
    const dim3 grid(n, H + 1);
    if (dtype == PL_DTYPE_F32) latent_prepare_kernel<float><<<grid, 64, 0, stream>>>(a);
    else if (dtype == PL_DTYPE_BF16) latent_prepare_kernel<bf16_t><<<grid, 64, 0, stream>>>(a);
    else PL_REQUIRE(false, "latent_prepare: dtype code %d", dtype);
    PL_CHECK_LAUNCH("latent_prepare");
    return 0;
}

// x[t, h, 0:V] *= sigmoid(g[t, h]): a gate a head on a read-out; g is 32-bit, column `g_off + h` of rows of `g_stride`.
// `each`: a gate an element instead, x[t, e] *= sigmoid(g[t, e]).
template <typename T>
__global__ __launch_bounds__(256) void head_gate_kernel(T* x, const float* g, int g_stride, int g_off, const int* positions,
                                                        int H, int V, int each) {
    const int t = blockIdx.x;
    if (positions != nullptr && positions[t] < 0) return;
    T* row = x + static_cast<size_t>(t) * H * V;
    const float* gates = g + static_cast<size_t>(t) * g_stride + g_off;
    for (int e = threadIdx.x; e < H * V; e += 256) {
        const float gate = 1.f / (1.f + expf(-gates[each ? e : e / V]));
        row[e] = from_float<T>(to_float(row[e]) * gate);
    }
}

extern "C" int pl_head_gate(void* x, int dtype, const float* g, int g_stride, int g_off, const int* positions, int n,
                            int H, int V, int each, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && H > 0 && V > 0 && g_off >= 0 && g_stride >= g_off + (each ? H * V : H), "head_gate: %d rows, %d heads of %d, gates at %d of %d", n, H, V, g_off, g_stride);
    if (n == 0) return 0;
    if (dtype == PL_DTYPE_F32) head_gate_kernel<float><<<n, 256, 0, stream>>>(static_cast<float*>(x), g, g_stride, g_off, positions, H, V, each);
    else if (dtype == PL_DTYPE_BF16) head_gate_kernel<bf16_t><<<n, 256, 0, stream>>>(static_cast<bf16_t*>(x), g, g_stride, g_off, positions, H, V, each);
    else PL_REQUIRE(false, "head_gate: dtype code %d", dtype);
    PL_CHECK_LAUNCH("head_gate");
    return 0;
}

// x[t] += table[positions[t]]: a learned vector a position on the 32-bit stream (rows at position -1 are padding).
template <typename T>
__global__ __launch_bounds__(256) void add_position_rows_kernel(float* x, const T* table, const int* positions, int width,
                                                                int table_rows) {
    const int t = blockIdx.x;
    const int pos = positions[t];
    if (pos < 0 || pos >= table_rows) return;
    float* row = x + static_cast<size_t>(t) * width;
    const T* add = table + static_cast<size_t>(pos) * width;
    for (int e = threadIdx.x; e < width; e += 256) row[e] += to_float(add[e]);
}

extern "C" int pl_add_position_rows(float* x, const void* table, int dtype, const int* positions, int n, int width,
                                    int table_rows, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && width > 0 && table_rows > 0, "add_position_rows: %d rows of %d, a table of %d", n, width, table_rows);
    if (n == 0) return 0;
    if (dtype == PL_DTYPE_F32) add_position_rows_kernel<float><<<n, 256, 0, stream>>>(x, static_cast<const float*>(table), positions, width, table_rows);
    else if (dtype == PL_DTYPE_BF16) add_position_rows_kernel<bf16_t><<<n, 256, 0, stream>>>(x, static_cast<const bf16_t*>(table), positions, width, table_rows);
    else PL_REQUIRE(false, "add_position_rows: dtype code %d", dtype);
    PL_CHECK_LAUNCH("add_position_rows");
    return 0;
}
