// A gated linear recurrence a channel (the real-gated linear recurrent unit) behind a short causal convolution:
//     u_t = bias + sum_j taps[j] * in_(t - (k - 1 - j))                       (zeros before a sequence's start;
//                                                                              taps are handed over as [k][width])
//     r_t = sigmoid(zr_t + br),  i_t = sigmoid(zi_t + bi)                    (zr, zi: block-diagonal products of u)
//     a_t = exp(-c * r_t * softplus(lam)),   S_t = a_t S_(t-1) + sqrt(1 - a_t^2) * i_t * u_t
//     out_t = S_t * gelu_tanh(branch_t)
// Gates, decays and the state are 32-bit.  What a request carries from step to step lies in its row of `state`,
// [slots][k][width] of 32-bit floats: row 0 the recurrent state S, rows 1..k-1 the last k - 1 inputs of the
// convolution, oldest first.  A new request's row is zero.
#include "api.h"
#include "common.h"

// u [n, width] (32-bit) of the step's tokens; reads the inputs that precede a request's portion from its state row.
template <typename T>
__global__ void conv_step_kernel(float* __restrict__ u, bf16_t* __restrict__ u_lo, const T* __restrict__ x, const T* __restrict__ taps,
                                 const T* __restrict__ bias, const float* __restrict__ state,
                                 const int* __restrict__ token_seq, const int* __restrict__ cu_tokens,
                                 const int* __restrict__ state_slots, int width, int k, long long x_ld, int x_off,
                                 long long total) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int t = (int)(i / width), c = (int)(i - (long long)t * width);
    const int seq = token_seq[t];
    const int first = cu_tokens[seq];
    const float* tail = state + ((long long)state_slots[seq] * k + 1) * width + c;      // rows 1..k-1
    float acc = bias != nullptr ? ld(bias + c) : 0.f;
    for (int j = 0; j < k; ++j) {
        const int src = t - (k - 1 - j);                    // the token this tap meets
        float v;
        if (src >= first) v = ld(x + (long long)src * x_ld + x_off + c);
        else v = tail[(long long)((k - 1) + (src - first)) * width];
        acc = fmaf(ld(taps + (long long)j * width + c), v, acc);
    }
    u[i] = acc;
    if (u_lo != nullptr) st(u_lo + i, acc);
}

// eight neighbouring bfloat16 values (16-byte aligned) as 32-bit floats
typedef uint32_t rec_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void unpack8(const bf16_t* p, float (&v)[8]) {
    const rec_u32x4 q = *reinterpret_cast<const rec_u32x4*>(p);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        v[2 * e] = __uint_as_float(q[e] << 16);
        v[2 * e + 1] = __uint_as_float(q[e] & 0xffff0000u);
    }
}

// The same for bfloat16 rows, eight neighbouring channels a thread (16-byte loads of the rows, two 16-byte stores of u
// and one of its bfloat16 copy): width, row length and offset in steps of 8.  The sums are those of the kernel above.
__global__ void conv_step8_kernel(float* __restrict__ u, bf16_t* __restrict__ u_lo, const bf16_t* __restrict__ x,
                                  const bf16_t* __restrict__ taps, const bf16_t* __restrict__ bias,
                                  const float* __restrict__ state, const int* __restrict__ token_seq,
                                  const int* __restrict__ cu_tokens, const int* __restrict__ state_slots, int width, int k,
                                  long long x_ld, int x_off, long long total8) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total8) return;
    const int per_row = width / 8;
    const int t = (int)(i / per_row), c = (int)(i - (long long)t * per_row) * 8;
    const int seq = token_seq[t];
    const int first = cu_tokens[seq];
    const float* tail = state + ((long long)state_slots[seq] * k + 1) * width + c;
    float acc[8];
    if (bias != nullptr) unpack8(bias + c, acc);
    else {
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    }
    for (int j = 0; j < k; ++j) {
        const int src = t - (k - 1 - j);
        float v[8], tp[8];
        unpack8(taps + (long long)j * width + c, tp);
        if (src >= first) {
            unpack8(x + (long long)src * x_ld + x_off + c, v);
        } else {
            const float* from = tail + (long long)((k - 1) + (src - first)) * width;
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = from[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = fmaf(tp[e], v[e], acc[e]);
    }
    float* out = u + (long long)t * width + c;
    *reinterpret_cast<float4*>(out) = make_float4(acc[0], acc[1], acc[2], acc[3]);
    *reinterpret_cast<float4*>(out + 4) = make_float4(acc[4], acc[5], acc[6], acc[7]);
    if (u_lo != nullptr) {
        uint4 q;
        q.x = pack_bf16x2(acc[0], acc[1]); q.y = pack_bf16x2(acc[2], acc[3]);
        q.z = pack_bf16x2(acc[4], acc[5]); q.w = pack_bf16x2(acc[6], acc[7]);
        *reinterpret_cast<uint4*>(u_lo + (long long)t * width + c) = q;
    }
}

// One thread a (request, channel) walks the request's tokens in order.  z [n, 2 * width] holds, block by block,
// [zr of the block | zi of the block] (blocks of `bw` channels).  Afterwards the thread moves the convolution's last
// inputs into the state row.
template <typename T>
__global__ void rglru_scan_kernel(T* __restrict__ out, float* __restrict__ state, const float* __restrict__ u,
                                  const float* __restrict__ z, const T* __restrict__ bias_r, const T* __restrict__ bias_i,
                                  const T* __restrict__ lam, const T* __restrict__ branch, const T* __restrict__ x,
                                  const int* __restrict__ cu_tokens, const int* __restrict__ state_slots, int width,
                                  int bw, int k, float decay, long long b_ld, int b_off, long long x_ld, int x_off) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= width) return;
    const int seq = blockIdx.y;
    const int first = cu_tokens[seq], last = cu_tokens[seq + 1];
    float* row = state + (long long)state_slots[seq] * k * width + c;
    const int blk = c / bw, j = c - blk * bw;
    const long long zr_at = (long long)blk * 2 * bw + j, zi_at = zr_at + bw;
    const float br = ld(bias_r + c), bi = ld(bias_i + c);
    const float l = ld(lam + c);
    const float sp = fmaxf(l, 0.f) + log1pf(expf(-fabsf(l)));             // softplus
    float S = row[0];
    for (int t = first; t < last; ++t) {
        const float r = 1.0f / (1.0f + expf(-(z[(long long)t * 2 * width + zr_at] + br)));
        const float g = 1.0f / (1.0f + expf(-(z[(long long)t * 2 * width + zi_at] + bi)));
        const float log_a = -decay * r * sp;
        const float a = expf(log_a);
        const float m = sqrtf(-expm1f(2.0f * log_a));                        // sqrt(1 - a^2)
        S = fmaf(a, S, m * g * u[(long long)t * width + c]);
        const float bv = ld(branch + (long long)t * b_ld + b_off + c);
        const float y = 0.5f * bv * (1.0f + tanhf(0.7978845608028654f * (bv + 0.044715f * bv * bv * bv)));
        st(out + (long long)t * width + c, S * y);
    }
    row[0] = S;
    // the last k - 1 inputs, oldest first: those of this portion, and before them what the row held
    const int q = last - first;
    for (int m = 0; m < k - 1; ++m) {
        const int src = last - (k - 1) + m;
        float v;
        if (src >= first) v = ld(x + (long long)src * x_ld + x_off + c);
        else v = row[(long long)(1 + m + q) * width];                       // (m + q < k - 1 here; read before it is written)
        row[(long long)(1 + m) * width] = v;
    }
}

extern "C" int ia_conv_step(float* u, void* u_lo, const void* x, const void* taps, const void* bias, const float* state,
                            const int* token_seq, const int* cu_tokens, const int* state_slots, int n, int width, int k,
                            long long x_ld, int x_off, int dtype, hipStream_t stream) {
    IA_CHECK(n >= 0 && width > 0 && k >= 1 && x_off >= 0 && x_off + width <= x_ld, "conv_step: bad sizes n=%d width=%d taps=%d",
             n, width, k);
    const long long total = (long long)n * width;
    if (total == 0) return 0;
    const int blocks = (int)((total + 255) / 256);
    if (dtype == IA_BF16 && width % 8 == 0 && x_ld % 8 == 0 && x_off % 8 == 0 && (((uintptr_t)x | (uintptr_t)u | (uintptr_t)u_lo) & 15) == 0) {
        const long long total8 = total / 8;
        conv_step8_kernel<<<(int)((total8 + 255) / 256), 256, 0, stream>>>(u, (bf16_t*)u_lo, (const bf16_t*)x, (const bf16_t*)taps,
                                                                          (const bf16_t*)bias, state, token_seq, cu_tokens,
                                                                          state_slots, width, k, x_ld, x_off, total8);
        IA_LAUNCH_CHECK("conv_step");
        return 0;
    }
    if (dtype == IA_F32)
        conv_step_kernel<float><<<blocks, 256, 0, stream>>>(u, (bf16_t*)u_lo, (const float*)x, (const float*)taps, (const float*)bias, state,
                                                            token_seq, cu_tokens, state_slots, width, k, x_ld, x_off, total);
    else
        conv_step_kernel<bf16_t><<<blocks, 256, 0, stream>>>(u, (bf16_t*)u_lo, (const bf16_t*)x, (const bf16_t*)taps, (const bf16_t*)bias,
                                                             state, token_seq, cu_tokens, state_slots, width, k, x_ld, x_off,
                                                             total);
    IA_LAUNCH_CHECK("conv_step");
    return 0;
}

extern "C" int ia_rglru_scan(void* out, float* state, const float* u, const float* z, const void* bias_r,
                             const void* bias_i, const void* lam, const void* branch, const void* x,
                             const int* cu_tokens, const int* state_slots, int n_seqs, int width, int bw, int k,
                             float decay, long long b_ld, int b_off, long long x_ld, int x_off, int dtype,
                             hipStream_t stream) {
    IA_CHECK(n_seqs >= 0 && width > 0 && bw > 0 && width % bw == 0 && k >= 1, "rglru_scan: bad sizes seqs=%d width=%d block=%d taps=%d",
             n_seqs, width, bw, k);
    IA_CHECK(b_off >= 0 && b_off + width <= b_ld && x_off >= 0 && x_off + width <= x_ld, "rglru_scan: the branches do not fit their rows");
    IA_CHECK(n_seqs <= 65535, "rglru_scan: %d requests are more than a grid takes", n_seqs);
    if (n_seqs == 0) return 0;
    const dim3 grid((width + 63) / 64, n_seqs);
    if (dtype == IA_F32)
        rglru_scan_kernel<float><<<grid, 64, 0, stream>>>((float*)out, state, u, z, (const float*)bias_r, (const float*)bias_i,
                                                          (const float*)lam, (const float*)branch, (const float*)x, cu_tokens,
                                                          state_slots, width, bw, k, decay, b_ld, b_off, x_ld, x_off);
    else
        rglru_scan_kernel<bf16_t><<<grid, 64, 0, stream>>>((bf16_t*)out, state, u, z, (const bf16_t*)bias_r,
                                                           (const bf16_t*)bias_i, (const bf16_t*)lam, (const bf16_t*)branch,
                                                           (const bf16_t*)x, cu_tokens, state_slots, width, bw, k, decay, b_ld,
                                                           b_off, x_ld, x_off);
    IA_LAUNCH_CHECK("rglru_scan");
    return 0;
}

// ---- the same recurrence for long portions: in chunks of 64 tokens side by side -----------------------------------
// S_t = a_t S_(t-1) + b_t is linear in the state a chunk starts from: with L_t the state reached from zero at the
// chunk's start and A_t the product of the chunk's decays up to t, S_t = L_t + A_t * S_in(chunk).  Three kernels:
// every chunk from zero (a thread a chunk and channel); a request's chunks in order (a thread a request and channel:
// S_in of the next chunk = L_end + A_end * S_in, then the state row and the convolution's last inputs); every token
// from its chunk's S_in.  The result differs from the token-by-token walk by rounding only.
#define IA_SCAN_CHUNK 64

// chunk g of the step -> its request and token range; requests own ceil(tokens / 64) chunks each, in order
__device__ __forceinline__ bool scan_chunk(const int* __restrict__ cu, int n_seqs, int g, int& seq, int& begin, int& end) {
    int at = 0;
    for (int s = 0; s < n_seqs; ++s) {
        const int first = cu[s], last = cu[s + 1];
        const int nc = (last - first + IA_SCAN_CHUNK - 1) / IA_SCAN_CHUNK;
        if (g < at + nc) {
            seq = s;
            begin = first + (g - at) * IA_SCAN_CHUNK;
            end = begin + IA_SCAN_CHUNK < last ? begin + IA_SCAN_CHUNK : last;
            return true;
        }
        at += nc;
    }
    return false;
}

template <typename T>
__global__ void rglru_chunks_kernel(float* __restrict__ loc, float* __restrict__ cum, float* __restrict__ chunk_a,
                                    float* __restrict__ chunk_l, int* __restrict__ token_chunk, const float* __restrict__ u,
                                    const float* __restrict__ z, const T* __restrict__ bias_r, const T* __restrict__ bias_i,
                                    const T* __restrict__ lam, const int* __restrict__ cu_tokens, int n_seqs, int width,
                                    int bw, float decay) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const int g = blockIdx.y;
    int seq, begin, end;
    if (!scan_chunk(cu_tokens, n_seqs, g, seq, begin, end)) return;
    if (blockIdx.x == 0)
        for (int t = begin + threadIdx.x; t < end; t += blockDim.x) token_chunk[t] = g;
    if (c >= width) return;
    const int blk = c / bw, j = c - blk * bw;
    const long long zr_at = (long long)blk * 2 * bw + j, zi_at = zr_at + bw;
    const float br = ld(bias_r + c), bi = ld(bias_i + c);
    const float l = ld(lam + c);
    const float sp = fmaxf(l, 0.f) + log1pf(expf(-fabsf(l)));
    float L = 0.f, A = 1.f;
    for (int t = begin; t < end; ++t) {
        const float r = 1.0f / (1.0f + expf(-(z[(long long)t * 2 * width + zr_at] + br)));
        const float gi = 1.0f / (1.0f + expf(-(z[(long long)t * 2 * width + zi_at] + bi)));
        const float log_a = -decay * r * sp;
        const float a = expf(log_a);
        const float m = sqrtf(-expm1f(2.0f * log_a));
        L = fmaf(a, L, m * gi * u[(long long)t * width + c]);
        A *= a;
        loc[(long long)t * width + c] = L;
        cum[(long long)t * width + c] = A;
    }
    chunk_a[(long long)g * width + c] = A;
    chunk_l[(long long)g * width + c] = L;
}

template <typename T>
__global__ void rglru_carry_kernel(float* __restrict__ chunk_in, float* __restrict__ state, const float* __restrict__ chunk_a,
                                   const float* __restrict__ chunk_l, const T* __restrict__ x,
                                   const int* __restrict__ cu_tokens, const int* __restrict__ state_slots, int width, int k,
                                   long long x_ld, int x_off) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= width) return;
    const int seq = blockIdx.y;
    int g = 0;
    for (int s = 0; s < seq; ++s) g += (cu_tokens[s + 1] - cu_tokens[s] + IA_SCAN_CHUNK - 1) / IA_SCAN_CHUNK;
    const int first = cu_tokens[seq], last = cu_tokens[seq + 1];
    const int nc = (last - first + IA_SCAN_CHUNK - 1) / IA_SCAN_CHUNK;
    float* row = state + (long long)state_slots[seq] * k * width + c;
    float S = row[0];
    for (int i = 0; i < nc; ++i) {
        const long long at = (long long)(g + i) * width + c;
        chunk_in[at] = S;
        S = fmaf(chunk_a[at], S, chunk_l[at]);
    }
    row[0] = S;
    const int q = last - first;
    for (int m = 0; m < k - 1; ++m) {
        const int src = last - (k - 1) + m;
        float v;
        if (src >= first) v = ld(x + (long long)src * x_ld + x_off + c);
        else v = row[(long long)(1 + m + q) * width];
        row[(long long)(1 + m) * width] = v;
    }
}

template <typename T>
__global__ void rglru_finish_kernel(T* __restrict__ out, const float* __restrict__ loc, const float* __restrict__ cum,
                                    const float* __restrict__ chunk_in, const int* __restrict__ token_chunk,
                                    const T* __restrict__ branch, int width, long long b_ld, int b_off, long long total) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int t = (int)(i / width), c = (int)(i - (long long)t * width);
    const float S = fmaf(cum[i], chunk_in[(long long)token_chunk[t] * width + c], loc[i]);
    const float bv = ld(branch + (long long)t * b_ld + b_off + c);
    const float y = 0.5f * bv * (1.0f + tanhf(0.7978845608028654f * (bv + 0.044715f * bv * bv * bv)));
    st(out + i, S * y);
}

// work: 2 n width + 3 chunks width floats and n ints, chunks = n / 64 + n_seqs (ia_rglru_chunked_workspace words)
extern "C" long long ia_rglru_chunked_workspace(int n, int n_seqs, int width) {
    const long long chunks = n / IA_SCAN_CHUNK + n_seqs;
    return 2LL * n * width + 3LL * chunks * width + n;
}

extern "C" int ia_rglru_scan_chunked(void* out, float* state, float* work, const float* u, const float* z,
                                     const void* bias_r, const void* bias_i, const void* lam, const void* branch,
                                     const void* x, const int* cu_tokens, const int* state_slots, int n, int n_seqs,
                                     int width, int bw, int k, float decay, long long b_ld, int b_off, long long x_ld,
                                     int x_off, int dtype, hipStream_t stream) {
    IA_CHECK(n >= 0 && n_seqs >= 0 && width > 0 && bw > 0 && width % bw == 0 && k >= 1, "rglru_scan_chunked: bad sizes");
    IA_CHECK(b_off >= 0 && b_off + width <= b_ld && x_off >= 0 && x_off + width <= x_ld, "rglru_scan_chunked: the branches do not fit their rows");
    if (n == 0 || n_seqs == 0) return 0;
    const int chunks = n / IA_SCAN_CHUNK + n_seqs;
    IA_CHECK(chunks <= 65535 && n_seqs <= 65535, "rglru_scan_chunked: %d chunks are more than a grid takes", chunks);
    float* loc = work;
    float* cum = loc + (long long)n * width;
    float* chunk_a = cum + (long long)n * width;
    float* chunk_l = chunk_a + (long long)chunks * width;
    float* chunk_in = chunk_l + (long long)chunks * width;
    int* token_chunk = (int*)(chunk_in + (long long)chunks * width);
    const dim3 g1((width + 63) / 64, chunks), g2((width + 63) / 64, n_seqs);
    const long long total = (long long)n * width;
    const int g3 = (int)((total + 255) / 256);
#define IA_RUN(T)                                                                                                       \
    rglru_chunks_kernel<T><<<g1, 64, 0, stream>>>(loc, cum, chunk_a, chunk_l, token_chunk, u, z, (const T*)bias_r,          \
                                                  (const T*)bias_i, (const T*)lam, cu_tokens, n_seqs, width, bw, decay);    \
    rglru_carry_kernel<T><<<g2, 64, 0, stream>>>(chunk_in, state, chunk_a, chunk_l, (const T*)x, cu_tokens, state_slots,    \
                                                 width, k, x_ld, x_off);                                                    \
    rglru_finish_kernel<T><<<g3, 256, 0, stream>>>((T*)out, loc, cum, chunk_in, token_chunk, (const T*)branch, width, b_ld, \
                                                   b_off, total)
    if (dtype == IA_F32) { IA_RUN(float); } else { IA_RUN(bf16_t); }
#undef IA_RUN
    IA_LAUNCH_CHECK("rglru_scan_chunked");
    return 0;
}
