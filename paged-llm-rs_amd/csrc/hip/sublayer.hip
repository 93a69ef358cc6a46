// What stands between the parts of a layer that normalises each sublayer's output instead of its input:
//   stream += rmsnorm(y) * gain     (with the updated rows again in the model's type, for the next part)
// and small passes over rows: a scale, a change of type, an activation, a weighted sum of two branches.
// The statistic, the gain and the sum into the stream are 32-bit.
#include "common.hpp"

template <typename T>
__global__ void rmsnorm_onto_kernel(float* __restrict__ resid, const float* __restrict__ y,
                                    const float* __restrict__ gain, float eps, T* __restrict__ rows_out, int H) {
    __shared__ float scratch[16];
    const size_t base = static_cast<size_t>(blockIdx.x) * H;
    float ss = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) ss += y[base + i] * y[base + i];
    ss = block_sum(ss, scratch);
    const float inv = 1.f / sqrtf(ss / static_cast<float>(H) + eps);
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        const float x = resid[base + i] + y[base + i] * inv * gain[i];
        resid[base + i] = x;
        if (rows_out != nullptr) rows_out[base + i] = from_float<T>(x);
    }
}

// rows_out may be null; its type is `dtype` otherwise.
extern "C" int pl_rmsnorm_onto(float* resid, const float* y, const float* gain, float eps, void* rows_out, int dtype,
                               int n, int H, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && H > 0, "rmsnorm_onto: rows %d, width %d", n, H);
    if (n == 0) return 0;
    const int threads = H >= 1024 ? 256 : (H >= 256 ? 128 : 64);
    if (rows_out == nullptr || dtype == PL_DTYPE_F32)
        rmsnorm_onto_kernel<float><<<n, threads, 0, stream>>>(resid, y, gain, eps, static_cast<float*>(rows_out), H);
    else if (dtype == PL_DTYPE_BF16)
        rmsnorm_onto_kernel<bf16_t><<<n, threads, 0, stream>>>(resid, y, gain, eps, static_cast<bf16_t*>(rows_out), H);
    else
        PL_REQUIRE(false, "rmsnorm_onto: dtype code %d", dtype);
    PL_CHECK_LAUNCH("rmsnorm_onto");
    return 0;
}

__global__ void scale_kernel(float* __restrict__ x, float s, size_t count) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < count) x[i] *= s;
}

extern "C" int pl_scale(float* x, float s, long count, hipStream_t stream) {
    PL_REQUIRE(count >= 0, "scale: %ld values", count);
    if (count == 0) return 0;
    scale_kernel<<<static_cast<unsigned>((count + 255) / 256), 256, 0, stream>>>(x, s, static_cast<size_t>(count));
    PL_CHECK_LAUNCH("scale");
    return 0;
}

__global__ void to_bf16_kernel(const float* __restrict__ x, bf16_t* __restrict__ out, size_t count) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < count) out[i] = from_float<bf16_t>(x[i]);
}

extern "C" int pl_to_bf16(const float* x, void* out, long count, hipStream_t stream) {
    PL_REQUIRE(count >= 0, "to_bf16: %ld values", count);
    if (count == 0) return 0;
    to_bf16_kernel<<<static_cast<unsigned>((count + 255) / 256), 256, 0, stream>>>(x, static_cast<bf16_t*>(out), static_cast<size_t>(count));
    PL_CHECK_LAUNCH("to_bf16");
    return 0;
}

// Eight values a thread where the count allows it (16 bytes of bfloat16, 32 of floats), one otherwise.
template <typename T, bool EXACT, int PER>
__global__ void activation_kernel(const T* __restrict__ x, T* __restrict__ out, int act, size_t count) {
    const size_t i = (static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x) * PER;
    if (i >= count) return;
    T in[PER], res[PER];
    if (PER == 8 && sizeof(T) == 2) {
        *reinterpret_cast<uint4*>(in) = *reinterpret_cast<const uint4*>(x + i);
    } else {
#pragma unroll
        for (int j = 0; j < PER; ++j) in[j] = x[i + j];
    }
#pragma unroll
    for (int j = 0; j < PER; ++j) res[j] = from_float<T>(pl_activate<EXACT>(to_float(in[j]), act));
    if (PER == 8 && sizeof(T) == 2) {
        *reinterpret_cast<uint4*>(out + i) = *reinterpret_cast<const uint4*>(res);
    } else {
#pragma unroll
        for (int j = 0; j < PER; ++j) out[i + j] = res[j];
    }
}

extern "C" int pl_activation(const void* x, void* out, int dtype, int act, long count, hipStream_t stream) {
    PL_REQUIRE(count >= 0 && act >= 0 && act <= 2, "activation: %ld values, code %d", count, act);
    if (count == 0) return 0;
    const bool eights = count % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
    const size_t items = eights ? count / 8 : count;
    const unsigned blocks = static_cast<unsigned>((items + 255) / 256);
    const size_t n = static_cast<size_t>(count);
    if (dtype == PL_DTYPE_F32) {
        if (eights) activation_kernel<float, true, 8><<<blocks, 256, 0, stream>>>(static_cast<const float*>(x), static_cast<float*>(out), act, n);
        else activation_kernel<float, true, 1><<<blocks, 256, 0, stream>>>(static_cast<const float*>(x), static_cast<float*>(out), act, n);
    } else if (dtype == PL_DTYPE_BF16) {
        if (eights) activation_kernel<bf16_t, true, 8><<<blocks, 256, 0, stream>>>(static_cast<const bf16_t*>(x), static_cast<bf16_t*>(out), act, n);
        else activation_kernel<bf16_t, true, 1><<<blocks, 256, 0, stream>>>(static_cast<const bf16_t*>(x), static_cast<bf16_t*>(out), act, n);
    } else {
        PL_REQUIRE(false, "activation: dtype code %d", dtype);
    }
    PL_CHECK_LAUNCH("activation");
    return 0;
}

__global__ void weighted_sum_kernel(float* __restrict__ x, float a, const float* __restrict__ y, float b, size_t count) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < count) x[i] = a * x[i] + b * y[i];
}

// x = a * x + b * y
extern "C" int pl_weighted_sum(float* x, float a, const float* y, float b, long count, hipStream_t stream) {
    PL_REQUIRE(count >= 0, "weighted_sum: %ld values", count);
    if (count == 0) return 0;
    weighted_sum_kernel<<<static_cast<unsigned>((count + 255) / 256), 256, 0, stream>>>(x, a, y, b, static_cast<size_t>(count));
    PL_CHECK_LAUNCH("weighted_sum");
    return 0;
}

// ---- a layer whose sublayers stand side by side -----------------------------------------------------------
//
// One pass over a row of the 32-bit stream, either half optional.  First the sums that are due,
//   x <- x + ls1 * a + ls2 * b + more
// (a, b: what the two sublayers of the layer before gave, 32-bit; ls1, ls2: a gain a column, or null for one; more: rows
// added as they are, e.g. what the model began with, before a stretch of layers runs again), written back to the stream.
// Then the norms that read the updated row: out1 = x / sqrt(mean(x^2) + eps) * gain1 and out2 likewise with gain2,
// rounded once into the model's type.  `rows` (with no sums due) names the rows to read.
struct ParallelStepArgs {
    float* resid;
    const float* a;
    const float* ls1;
    const float* b;
    const float* ls2;
    const float* more;
    const float* gain1;
    const float* gain2;
    float eps;
    void* out1;
    void* out2;
    const int* rows;
    int W;
};

template <int PER>
struct Run {
    float v[PER];
};

template <int PER>
__device__ __forceinline__ Run<PER> load_run(const float* p) {
    Run<PER> r;
    if (PER == 4) {
        const float4 q = *reinterpret_cast<const float4*>(p);
        r.v[0] = q.x;
        r.v[1 % PER] = q.y;
        r.v[2 % PER] = q.z;
        r.v[3 % PER] = q.w;
    } else {
        r.v[0] = p[0];
    }
    return r;
}

template <int PER>
__device__ __forceinline__ void store_run(float* p, const Run<PER>& r) {
    if (PER == 4) *reinterpret_cast<float4*>(p) = make_float4(r.v[0], r.v[1 % PER], r.v[2 % PER], r.v[3 % PER]);
    else p[0] = r.v[0];
}

template <int PER>
__device__ __forceinline__ void store_run(bf16_t* p, const Run<PER>& r) {
    if (PER == 4) {
        uint2 w;
        w.x = static_cast<uint32_t>(bf16_bits_from_float(r.v[0])) | (static_cast<uint32_t>(bf16_bits_from_float(r.v[1 % PER])) << 16);
        w.y = static_cast<uint32_t>(bf16_bits_from_float(r.v[2 % PER])) | (static_cast<uint32_t>(bf16_bits_from_float(r.v[3 % PER])) << 16);
        *reinterpret_cast<uint2*>(p) = w;
    } else {
        p[0] = from_float<bf16_t>(r.v[0]);
    }
}

// A workgroup a row; a thread takes runs of PER columns.  A thread's first run stays in registers between the two
// halves (rows up to PER * blockDim columns are read once), further ones are read back from the stream.
template <typename T, int PER>
__global__ __launch_bounds__(1024) void parallel_step_kernel(ParallelStepArgs p) {
    __shared__ float scratch[16];
    const int i = blockIdx.x, W = p.W;
    const size_t in_row = static_cast<size_t>(p.rows != nullptr ? p.rows[i] : i) * W;
    const size_t out_row = static_cast<size_t>(i) * W;
    float* x = p.resid + in_row;
    const bool sums = p.a != nullptr || p.b != nullptr || p.more != nullptr;
    Run<PER> first;
    float ss = 0.f;
    for (int c = threadIdx.x * PER; c < W; c += blockDim.x * PER) {
        Run<PER> v = load_run<PER>(x + c);
        if (p.a != nullptr) {
            const Run<PER> y = load_run<PER>(p.a + in_row + c);
            if (p.ls1 != nullptr) {
                const Run<PER> g = load_run<PER>(p.ls1 + c);
#pragma unroll
                for (int j = 0; j < PER; ++j) v.v[j] += y.v[j] * g.v[j];
            } else {
#pragma unroll
                for (int j = 0; j < PER; ++j) v.v[j] += y.v[j];
            }
        }
        if (p.b != nullptr) {
            const Run<PER> y = load_run<PER>(p.b + in_row + c);
            if (p.ls2 != nullptr) {
                const Run<PER> g = load_run<PER>(p.ls2 + c);
#pragma unroll
                for (int j = 0; j < PER; ++j) v.v[j] += y.v[j] * g.v[j];
            } else {
#pragma unroll
                for (int j = 0; j < PER; ++j) v.v[j] += y.v[j];
            }
        }
        if (p.more != nullptr) {
            const Run<PER> y = load_run<PER>(p.more + in_row + c);
#pragma unroll
            for (int j = 0; j < PER; ++j) v.v[j] += y.v[j];
        }
        if (sums) store_run<PER>(x + c, v);
#pragma unroll
        for (int j = 0; j < PER; ++j) ss += v.v[j] * v.v[j];
        if (c == static_cast<int>(threadIdx.x) * PER) first = v;
    }
    if (p.gain1 == nullptr) return;
    ss = block_sum(ss, scratch);
    const float inv = 1.f / sqrtf(ss / static_cast<float>(W) + p.eps);
    T* out1 = static_cast<T*>(p.out1) + out_row;
    T* out2 = p.gain2 != nullptr ? static_cast<T*>(p.out2) + out_row : nullptr;
    for (int c = threadIdx.x * PER; c < W; c += blockDim.x * PER) {
        const Run<PER> v = c == static_cast<int>(threadIdx.x) * PER ? first : load_run<PER>(x + c);
        const Run<PER> g1 = load_run<PER>(p.gain1 + c);
        Run<PER> o;
#pragma unroll
        for (int j = 0; j < PER; ++j) o.v[j] = v.v[j] * inv * g1.v[j];
        store_run<PER>(out1 + c, o);
        if (out2 != nullptr) {
            const Run<PER> g2 = load_run<PER>(p.gain2 + c);
#pragma unroll
            for (int j = 0; j < PER; ++j) o.v[j] = v.v[j] * inv * g2.v[j];
            store_run<PER>(out2 + c, o);
        }
    }
}

extern "C" int pl_parallel_step(float* resid, const float* a, const float* ls1, const float* b, const float* ls2,
                                const float* more, const float* gain1, const float* gain2, float eps, void* out1, void* out2,
                                int dtype, const int* rows, int n, int W, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && W > 0, "parallel_step: rows %d, width %d", n, W);
    PL_REQUIRE(rows == nullptr || (a == nullptr && b == nullptr && more == nullptr), "parallel_step: a list of rows and sums into the stream");
    PL_REQUIRE((gain1 != nullptr || gain2 == nullptr) && (gain1 == nullptr || out1 != nullptr) && (gain2 == nullptr || out2 != nullptr),
               "parallel_step: a second norm without a first, or a norm without room for its rows");
    PL_REQUIRE(dtype == PL_DTYPE_F32 || dtype == PL_DTYPE_BF16, "parallel_step: dtype code %d", dtype);
    if (n == 0) return 0;
    ParallelStepArgs p{resid, a, ls1, b, ls2, more, gain1, gain2, eps, out1, out2, rows, W};
    if (W % 4 == 0) {
        int threads = ((W / 4 + 63) / 64) * 64;
        threads = threads > 1024 ? 1024 : threads;
        if (dtype == PL_DTYPE_F32) parallel_step_kernel<float, 4><<<n, threads, 0, stream>>>(p);
        else parallel_step_kernel<bf16_t, 4><<<n, threads, 0, stream>>>(p);
    } else {
        const int threads = W >= 1024 ? 256 : (W >= 256 ? 128 : 64);
        if (dtype == PL_DTYPE_F32) parallel_step_kernel<float, 1><<<n, threads, 0, stream>>>(p);
        else parallel_step_kernel<bf16_t, 1><<<n, threads, 0, stream>>>(p);
    }
    PL_CHECK_LAUNCH("parallel_step");
    return 0;
}
