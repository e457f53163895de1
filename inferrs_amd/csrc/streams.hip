// Several residual streams a token (hyper-connections), kept in 32-bit: `streams` is [tokens, S, width].
//
// One kernel does what stands between two sub-layers.  With the output y of the sub-layer that has just run,
//     x_t <- sum_s mix[s][t] x_s + out[t] * scale[c] * y[c]        (all streams at once from the old ones)
// and then, for the sub-layer that runs next,
//     h = rmsnorm(sum_s in[s] x_s) * w
// in the precision of that sub-layer's products.  Either half may be absent (the first read of a step has no y;
// the last write of a model is followed by a read of the wanted rows only).  y may be the weighted sum of K rows a
// token (the outputs of a token's K routed experts, weights in 32-bit), added up in the order of k.
// S = 1 with mix = out = in = 1 is the ordinary residual sum with a per-feature scale, in 32-bit.
// A block owns a row; sums of squares in 32-bit.
#include "api.h"
#include "common.h"

#define IA_MAX_STREAMS 8

template <typename TY, typename TH>
__global__ __launch_bounds__(512) void streams_step_kernel(
    float* __restrict__ streams, const TY* __restrict__ y, const float* __restrict__ yw, int K,
    const float* __restrict__ scale, const float* __restrict__ mix, const float* __restrict__ outc,
    const float* __restrict__ inc, const float* __restrict__ w, float eps, TH* __restrict__ h,
    const int* __restrict__ rows, int S, int W) {
    extern __shared__ float u_sh[];              // [W]: the row that the norm reads
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int row = rows != nullptr ? rows[r] : r;
    // (the coefficients are the same for every lane: read where they are used, they come through the scalar cache
    // beside the row's own loads instead of a round trip ahead of them)
    const float* cm = mix;                       // [S][S]
    const float* co = outc;
    float* xr = streams + (long long)row * S * W;
    float sq = 0.f;
#pragma unroll 4
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        float x[IA_MAX_STREAMS];
#pragma unroll
        for (int s = 0; s < IA_MAX_STREAMS; ++s) x[s] = s < S ? xr[(long long)s * W + c] : 0.f;
        if (y != nullptr) {
            float yv;
            if (yw != nullptr) {
                yv = 0.f;
                for (int k = 0; k < K; ++k)
                    yv = fmaf(yw[(long long)row * K + k], ld(y + ((long long)row * K + k) * W + c), yv);
            } else {
                yv = ld(y + (long long)row * W + c);
            }
            if (scale != nullptr) yv *= scale[c];
            float nx[IA_MAX_STREAMS];
#pragma unroll
            for (int t = 0; t < IA_MAX_STREAMS; ++t) {
                float v = 0.f;
                if (t < S) {
                    for (int s = 0; s < S; ++s) v = fmaf(cm[s * S + t], x[s], v);
                    v = fmaf(co[t], yv, v);
                    xr[(long long)t * W + c] = v;
                }
                nx[t] = v;
            }
#pragma unroll
            for (int t = 0; t < IA_MAX_STREAMS; ++t) x[t] = nx[t];
        }
        if (h != nullptr) {
            float u = 0.f;
#pragma unroll
            for (int s = 0; s < IA_MAX_STREAMS; ++s)
                if (s < S) u = fmaf(inc != nullptr ? inc[s] : 1.f, x[s], u);
            u_sh[c] = u;
            sq = fmaf(u, u, sq);
        }
    }
    if (h == nullptr) return;
    const float total = block_sum(sq, scratch);
    const float rs = 1.0f / sqrtf(total / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float v = u_sh[c] * rs;
        st(h + (long long)r * W + c, w != nullptr ? v * w[c] : v);
    }
}

// The same for rows of up to 4,096 features: a thread owns up to four columns and asks for everything it reads (the
// streams, the output, scales, the norm's weight) before it stores anything, so that one trip to the memory serves the
// whole step; the kernel above updates the streams in place column by column, and a column's loads cannot pass the
// stores of the column before.  The arithmetic and its order are those of the kernel above.
#define IA_STREAMS_COLS 4

template <typename TY, typename TH>
__global__ __launch_bounds__(1024) void streams_step_rows_kernel(
    float* __restrict__ streams, const TY* __restrict__ y, const float* __restrict__ yw, int K,
    const float* __restrict__ scale, const float* __restrict__ mix, const float* __restrict__ outc,
    const float* __restrict__ inc, const float* __restrict__ w, float eps, TH* __restrict__ h,
    const int* __restrict__ rows, int S, int W) {
    __shared__ float scratch[16];
    const int r = blockIdx.x, tid = threadIdx.x, nt = blockDim.x;
    const int row = rows != nullptr ? rows[r] : r;
    float* xr = streams + (long long)row * S * W;
    float x[IA_STREAMS_COLS][IA_MAX_STREAMS], yv[IA_STREAMS_COLS], wn[IA_STREAMS_COLS];
#pragma unroll
    for (int i = 0; i < IA_STREAMS_COLS; ++i) {
        const int c = tid + i * nt;
        const bool in = c < W;
#pragma unroll
        for (int s = 0; s < IA_MAX_STREAMS; ++s) x[i][s] = (in && s < S) ? xr[(long long)s * W + c] : 0.f;
        yv[i] = 0.f;
        if (y != nullptr && in) {
            if (yw != nullptr) {
                for (int k = 0; k < K; ++k)
                    yv[i] = fmaf(yw[(long long)row * K + k], ld(y + ((long long)row * K + k) * W + c), yv[i]);
            } else {
                yv[i] = ld(y + (long long)row * W + c);
            }
            if (scale != nullptr) yv[i] *= scale[c];
        }
        wn[i] = (h != nullptr && w != nullptr && in) ? w[c] : 1.f;
    }
    float u[IA_STREAMS_COLS];
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < IA_STREAMS_COLS; ++i) {
        const int c = tid + i * nt;
        const bool in = c < W;
        if (y != nullptr) {
            float nx[IA_MAX_STREAMS];
#pragma unroll
            for (int t = 0; t < IA_MAX_STREAMS; ++t) {
                float v = 0.f;
                if (t < S) {
                    for (int s = 0; s < S; ++s) v = fmaf(mix[s * S + t], x[i][s], v);
                    v = fmaf(outc[t], yv[i], v);
                    if (in) xr[(long long)t * W + c] = v;
                }
                nx[t] = v;
            }
#pragma unroll
            for (int t = 0; t < IA_MAX_STREAMS; ++t) x[i][t] = nx[t];
        }
        u[i] = 0.f;
#pragma unroll
        for (int s = 0; s < IA_MAX_STREAMS; ++s)
            if (s < S) u[i] = fmaf(inc != nullptr ? inc[s] : 1.f, x[i][s], u[i]);
        if (in) sq = fmaf(u[i], u[i], sq);
    }
    if (h == nullptr) return;
    const float total = block_sum(sq, scratch);
    const float rs = 1.0f / sqrtf(total / (float)W + eps);
#pragma unroll
    for (int i = 0; i < IA_STREAMS_COLS; ++i) {
        const int c = tid + i * nt;
        if (c < W) st(h + (long long)r * W + c, u[i] * rs * wn[i]);
    }
}

// y_dtype / h_dtype: 0 float32, 1 bfloat16.  y null: nothing is written to the streams; h null: nothing is read for
// a next sub-layer.  rows null: every row 0..n-1; else the n rows named (only for a call without y).
extern "C" int ia_streams_step(float* streams, const void* y, const float* yw, int K, const float* scale,
                               const float* mix, const float* outc, const float* inc, const float* w, float eps,
                               void* h, const int* rows, int n, int S, int W, int y_dtype, int h_dtype,
                               hipStream_t stream) {
    IA_CHECK(n >= 0 && W > 0 && S >= 1 && S <= IA_MAX_STREAMS, "streams_step: n=%d width=%d streams=%d (1..%d)", n, W, S,
             IA_MAX_STREAMS);
    IA_CHECK(y == nullptr || (mix != nullptr && outc != nullptr), "streams_step: an output to add needs mix and out");
    IA_CHECK(y == nullptr || rows == nullptr, "streams_step: a row list goes with a read only");
    IA_CHECK(K >= 1, "streams_step: K=%d", K);
    IA_CHECK((size_t)W * sizeof(float) <= 60 * 1024, "streams_step: width %d does not fit shared memory", W);
    if (n == 0 || (y == nullptr && h == nullptr)) return 0;
    const size_t shm = h != nullptr ? (size_t)W * sizeof(float) : 0;
    const int threads = W >= 2048 ? 512 : 256;
    const bool few = W <= 1024 * IA_STREAMS_COLS;
    const int row_threads = ((W + IA_STREAMS_COLS - 1) / IA_STREAMS_COLS + 63) / 64 * 64;
#define IA_LAUNCH(TY, TH)                                                                                              \
    if (few)                                                                                                           \
        streams_step_rows_kernel<TY, TH><<<n, row_threads, 0, stream>>>(streams, (const TY*)y, yw, K, scale, mix, outc,   \
                                                                        inc, w, eps, (TH*)h, rows, S, W);                \
    else                                                                                                               \
        streams_step_kernel<TY, TH><<<n, threads, shm, stream>>>(streams, (const TY*)y, yw, K, scale, mix, outc, inc, w,  \
                                                                 eps, (TH*)h, rows, S, W)
    if (y_dtype == IA_F32 && h_dtype == IA_F32) { IA_LAUNCH(float, float); }
    else if (y_dtype == IA_F32) { IA_LAUNCH(float, bf16_t); }
    else if (h_dtype == IA_F32) { IA_LAUNCH(bf16_t, float); }
    else { IA_LAUNCH(bf16_t, bf16_t); }
#undef IA_LAUNCH
    IA_LAUNCH_CHECK("streams_step");
    return 0;
}

// rows of the stream's width copied into every stream of a token: streams[t][s][:] = x[t][:]
template <typename T>
__global__ void streams_open_kernel(float* __restrict__ streams, const T* __restrict__ x, int S, int W, long long total) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const long long t = i / W;
    const int c = (int)(i - t * W);
    const float v = ld(x + i);
    for (int s = 0; s < S; ++s) streams[(t * S + s) * W + c] = v;
}

extern "C" int ia_streams_open(float* streams, const void* x, int n, int S, int W, int dtype, hipStream_t stream) {
    IA_CHECK(n >= 0 && W > 0 && S >= 1, "streams_open: n=%d width=%d streams=%d", n, W, S);
    const long long total = (long long)n * W;
    if (total == 0) return 0;
    const int blocks = (int)((total + 255) / 256);
    if (dtype == IA_F32) streams_open_kernel<float><<<blocks, 256, 0, stream>>>(streams, (const float*)x, S, W, total);
    else streams_open_kernel<bf16_t><<<blocks, 256, 0, stream>>>(streams, (const bf16_t*)x, S, W, total);
    IA_LAUNCH_CHECK("streams_open");
    return 0;
}

// logits <- cap * tanh(logits / cap), in place
__global__ void softcap_kernel(float* __restrict__ x, float cap, long long n) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

extern "C" int ia_softcap(float* x, long long n, float cap, hipStream_t stream) {
    IA_CHECK(n >= 0 && cap > 0.f, "softcap: n=%lld cap=%g", n, (double)cap);
    if (n == 0) return 0;
    softcap_kernel<<<(int)((n + 255) / 256), 256, 0, stream>>>(x, cap, n);
    IA_LAUNCH_CHECK("softcap");
    return 0;
}
