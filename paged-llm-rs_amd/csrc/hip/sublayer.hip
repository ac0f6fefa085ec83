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
