// A residual stream kept in 32-bit whose sub-layers stand between two norms:
//     x <- x + rmsnorm(y) * w_post,      y = s1 * y1 (+ s2 * y2)      (the sub-layer's output, or two outputs side by side; eps_post)
//     x <- x + e_rows + e_vec                                         (optional: a row and a vector that enter the stream here)
//     h  = rmsnorm(x) * w_pre                                         (the next sub-layer's input, in its products' precision)
// ONE kernel does what stands between two sub-layers; every half may be absent.  A block owns a row; sums of squares,
// the stream and its sums are 32-bit.  With `rows` the kernel reads the named rows only and writes nothing back to the
// stream (the model's end: the wanted rows through the final norm).
#include "api.h"
#include "common.h"

template <typename TY, typename TH>
__global__ __launch_bounds__(1024) void sandwich_step_kernel(
    float* __restrict__ x, const TY* __restrict__ y1, float s1, const TY* __restrict__ y2, float s2,
    const float* __restrict__ w_post, const TY* __restrict__ e_rows, const float* __restrict__ e_vec,
    const float* __restrict__ w_pre, float eps_post, float eps, TH* __restrict__ h, const int* __restrict__ rows, int W) {
    extern __shared__ float sw_row[];            // [W]
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int row = rows != nullptr ? rows[r] : r;
    float* xr = x + (long long)row * W;
    float rs = 0.f;
    if (y1 != nullptr) {
        float sq = 0.f;
        for (int c = threadIdx.x; c < W; c += blockDim.x) {
            float v = s1 * ld(y1 + (long long)row * W + c);
            if (y2 != nullptr) v = fmaf(s2, ld(y2 + (long long)row * W + c), v);
            sw_row[c] = v;
            sq = fmaf(v, v, sq);
        }
        rs = 1.0f / sqrtf(block_sum(sq, scratch) / (float)W + eps_post);
    }
    float sq = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        float v = xr[c];
        if (y1 != nullptr) v += sw_row[c] * rs * w_post[c];
        if (e_rows != nullptr) v += ld(e_rows + (long long)row * W + c);
        if (e_vec != nullptr) v += e_vec[c];
        if (rows == nullptr && (y1 != nullptr || e_rows != nullptr || e_vec != nullptr)) xr[c] = v;
        sw_row[c] = v;
        sq = fmaf(v, v, sq);
    }
    if (h == nullptr) return;
    const float rs2 = 1.0f / sqrtf(block_sum(sq, scratch) / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += blockDim.x)
        st(h + (long long)r * W + c, sw_row[c] * rs2 * (w_pre != nullptr ? w_pre[c] : 1.f));
}

// y_dtype: precision of y1, y2 and e_rows; h_dtype: of h.  0 float32, 1 bfloat16.
extern "C" int ia_sandwich_step(float* x, const void* y1, float s1, const void* y2, float s2, const float* w_post,
                                const void* e_rows, const float* e_vec, const float* w_pre, float eps_post, float eps, void* h,
                                const int* rows, int n, int W, int y_dtype, int h_dtype, hipStream_t stream) {
    IA_CHECK(n >= 0 && W > 0, "sandwich_step: n=%d width=%d", n, W);
    IA_CHECK((size_t)W * sizeof(float) <= 60 * 1024, "sandwich_step: width %d does not fit shared memory", W);
    IA_CHECK(y1 != nullptr || y2 == nullptr, "sandwich_step: a second output goes with a first");
    IA_CHECK(y1 == nullptr || w_post != nullptr, "sandwich_step: an output to add needs the weight of the norm behind it");
    if (n == 0) return 0;
    const int threads = W >= 4096 ? 1024 : W >= 1024 ? 512 : 256;
    const size_t shm = (size_t)W * sizeof(float);
#define IA_LAUNCH(TY, TH)                                                                                         \
    sandwich_step_kernel<TY, TH><<<n, threads, shm, stream>>>(x, (const TY*)y1, s1, (const TY*)y2, s2, w_post,      \
                                                              (const TY*)e_rows, e_vec, w_pre, eps_post, eps, (TH*)h, rows, W)
    if (y_dtype == IA_F32 && h_dtype == IA_F32) { IA_LAUNCH(float, float); }
    else if (y_dtype == IA_F32) { IA_LAUNCH(float, bf16_t); }
    else if (h_dtype == IA_F32) { IA_LAUNCH(bf16_t, float); }
    else { IA_LAUNCH(bf16_t, bf16_t); }
#undef IA_LAUNCH
    IA_LAUNCH_CHECK("sandwich_step");
    return 0;
}

__device__ __forceinline__ float act_value(float z, int act) {
    return act == 3 ? 0.5f * z * (1.0f + erff(z * 0.7071067811865476f)) : gate_act(z, act);
}

// An activation over every element, in place.  act: 1 SiLU, 2 GELU in its tanh form, 3 the exact GELU,
// z / 2 * (1 + erf(z / sqrt 2)).
template <typename T>
__global__ void activation_kernel(T* __restrict__ x, long long n, int act) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float z = ld(x + i);
    st(x + i, act_value(z, act));
}

// Eight neighbouring bfloat16 values a thread (16-byte accesses), for arrays of a multiple of eight elements.
__global__ void activation8_kernel(bf16_t* __restrict__ x, long long n8, int act) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n8) return;
    uint4 q = *reinterpret_cast<const uint4*>(x + 8 * i);
    uint32_t* w = reinterpret_cast<uint32_t*>(&q);
#pragma unroll
    for (int e = 0; e < 4; ++e)
        w[e] = pack_bf16x2(act_value(__uint_as_float(w[e] << 16), act), act_value(__uint_as_float(w[e] & 0xffff0000u), act));
    *reinterpret_cast<uint4*>(x + 8 * i) = q;
}

extern "C" int ia_activation(void* x, long long n, int act, int dtype, hipStream_t stream) {
    IA_CHECK(n >= 0 && act >= 1 && act <= 3, "activation: n=%lld act=%d (1 SiLU, 2 GELU tanh, 3 GELU)", n, act);
    if (n == 0) return 0;
    if (dtype != IA_F32 && n % 8 == 0 && ((uintptr_t)x & 15) == 0) {
        activation8_kernel<<<(unsigned)((n / 8 + 255) / 256), 256, 0, stream>>>((bf16_t*)x, n / 8, act);
        IA_LAUNCH_CHECK("activation");
        return 0;
    }
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (dtype == IA_F32) activation_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, n, act);
    else activation_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)x, n, act);
    IA_LAUNCH_CHECK("activation");
    return 0;
}
