// Mixers that carry a matrix of fixed size a head from token to token (linear attention in its recurrent form):
//     S_t = a_t S_(t-1) + b_t k_t v_t^T,      o_t = S_t^T q_t (+ skip * v_t)            S: [dim x vdim], 32-bit
// with a decay a_t and an input scale b_t that are scalars a (token, head).  Three mixers are this with other gates:
//   * retention: a a constant of the head, b = 1;
//   * the matrix memory with exponential gates: a = exp(f + m_(t-1) - m_t), b = exp(i - m_t) under a running maximum
//     m_t = max(f + m_(t-1), i); its normaliser n_t = a n_(t-1) + b k_t is the same recurrence with a value that is
//     always 1, carried here as one more column of S, whose output is n_t . q_t;
//   * the selective state space: a = exp(-exp(A) dt), b = dt, k = B, v = x, q = C, skip = D.
// The state, the decays, their logarithms and every sum are 32-bit; q, k and v come out of the projections (and a
// short convolution) in the products' precision.
//
// What a request carries lies in its row of a 32-bit state array [slots][row_floats]; the kernels take the offset of
// their part of the row: the matrices as [head][column j of S, vdim (+ 1)][dim], the running maxima [head], a
// convolution's last inputs [taps - 1][channels], oldest first.  A new request's row is zero.
#include "api.h"
#include "common.h"

// ---- a short causal convolution a channel, with its activation -----------------------------------------------------
// out[t][c] = act(bias[c] + sum_j taps[j][c] * in_(t - (k - 1 - j))[c]); inputs before the portion come from the tail.
template <typename T>
__global__ void conv_act_kernel(T* __restrict__ out, const T* __restrict__ x, const T* __restrict__ taps,
                                const T* __restrict__ bias, const float* __restrict__ state, long long row_floats,
                                long long tail_off, const int* __restrict__ token_seq, const int* __restrict__ cu_tokens,
                                const int* __restrict__ state_slots, int C, int k, long long x_ld, int x_off, int act,
                                long long total) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int t = (int)(i / C), c = (int)(i - (long long)t * C);
    const int seq = token_seq[t];
    const int first = cu_tokens[seq];
    const float* tail = state + (long long)state_slots[seq] * row_floats + tail_off + c;      // [k - 1][C]
    float acc = bias != nullptr ? ld(bias + c) : 0.f;
    for (int j = 0; j < k; ++j) {
        const int src = t - (k - 1 - j);
        float v;
        if (src >= first) v = ld(x + (long long)src * x_ld + x_off + c);
        else v = tail[(long long)((k - 1) + (src - first)) * C];
        acc = fmaf(ld(taps + (long long)j * C + c), v, acc);
    }
    if (act == IA_ACT_SILU) acc = acc / (1.0f + expf(-acc));
    st(out + i, acc);
}

// The same for bfloat16 rows, eight neighbouring channels a thread (16-byte accesses): channels, row length and
// offset in steps of 8.  The sums are those of the kernel above.
typedef uint32_t ls_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void ls_unpack8(const bf16_t* p, float (&v)[8]) {
    const ls_u32x4 q = *reinterpret_cast<const ls_u32x4*>(p);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        v[2 * e] = __uint_as_float(q[e] << 16);
        v[2 * e + 1] = __uint_as_float(q[e] & 0xffff0000u);
    }
}

__global__ void conv_act8_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ x, const bf16_t* __restrict__ taps,
                                 const bf16_t* __restrict__ bias, const float* __restrict__ state, long long row_floats,
                                 long long tail_off, const int* __restrict__ token_seq, const int* __restrict__ cu_tokens,
                                 const int* __restrict__ state_slots, int C, int k, long long x_ld, int x_off, int act,
                                 long long total8) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total8) return;
    const int per_row = C / 8;
    const int t = (int)(i / per_row), c = (int)(i - (long long)t * per_row) * 8;
    const int seq = token_seq[t];
    const int first = cu_tokens[seq];
    const float* tail = state + (long long)state_slots[seq] * row_floats + tail_off + c;
    float acc[8];
    if (bias != nullptr) ls_unpack8(bias + c, acc);
    else {
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    }
    for (int j = 0; j < k; ++j) {
        const int src = t - (k - 1 - j);
        float v[8], tp[8];
        ls_unpack8(taps + (long long)j * C + c, tp);
        if (src >= first) {
            ls_unpack8(x + (long long)src * x_ld + x_off + c, v);
        } else {
            const float* from = tail + (long long)((k - 1) + (src - first)) * C;
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = from[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = fmaf(tp[e], v[e], acc[e]);
    }
    if (act == IA_ACT_SILU) {
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = acc[e] / (1.0f + expf(-acc[e]));
    }
    ls_u32x4 q;
    q[0] = pack_bf16x2(acc[0], acc[1]); q[1] = pack_bf16x2(acc[2], acc[3]);
    q[2] = pack_bf16x2(acc[4], acc[5]); q[3] = pack_bf16x2(acc[6], acc[7]);
    *reinterpret_cast<ls_u32x4*>(out + (long long)t * C + c) = q;
}

// After the convolution of a step: a request's tail takes the last k - 1 inputs, oldest first.
template <typename T>
__global__ void conv_tail_kernel(float* __restrict__ state, long long row_floats, long long tail_off,
                                 const T* __restrict__ x, const int* __restrict__ cu_tokens,
                                 const int* __restrict__ state_slots, int C, int k, long long x_ld, int x_off) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int seq = blockIdx.y;
    const int first = cu_tokens[seq], last = cu_tokens[seq + 1];
    float* tail = state + (long long)state_slots[seq] * row_floats + tail_off + c;
    const int q = last - first;
    for (int m = 0; m < k - 1; ++m) {
        const int src = last - (k - 1) + m;
        float v;
        if (src >= first) v = ld(x + (long long)src * x_ld + x_off + c);
        else v = tail[(long long)(m + q) * C];                              // (m + q < k - 1 here; read before it is written)
        tail[(long long)m * C] = v;
    }
}

extern "C" int ia_conv_act_step(void* out, const void* x, const void* taps, const void* bias, float* state,
                                long long row_floats, long long tail_off, const int* token_seq, const int* cu_tokens,
                                const int* state_slots, int n, int n_seqs, int C, int k, long long x_ld, int x_off, int act,
                                int dtype, hipStream_t stream) {
    IA_CHECK(n >= 0 && n_seqs >= 0 && C > 0 && k >= 1 && x_off >= 0 && x_off + C <= x_ld,
             "conv_act_step: bad sizes n=%d channels=%d taps=%d", n, C, k);
    IA_CHECK(tail_off >= 0 && tail_off + (long long)(k - 1) * C <= row_floats, "conv_act_step: the tail does not fit the state row");
    IA_CHECK(act == IA_ACT_NONE || act == IA_ACT_SILU, "conv_act_step: activation %d (0 none, 1 SiLU)", act);
    if (n == 0 || n_seqs == 0) return 0;
    const long long total = (long long)n * C;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    const dim3 tail_grid((unsigned)((C + 255) / 256), (unsigned)n_seqs);
    if (dtype == IA_F32) {
        conv_act_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, (const float*)x, (const float*)taps, (const float*)bias,
                                                           state, row_floats, tail_off, token_seq, cu_tokens, state_slots, C, k,
                                                           x_ld, x_off, act, total);
        if (k > 1)
            conv_tail_kernel<float><<<tail_grid, 256, 0, stream>>>(state, row_floats, tail_off, (const float*)x, cu_tokens,
                                                                   state_slots, C, k, x_ld, x_off);
    } else {
        const bool wide = C % 8 == 0 && x_ld % 8 == 0 && x_off % 8 == 0 && tail_off % 4 == 0 && row_floats % 4 == 0 &&
                          (((uintptr_t)out | (uintptr_t)x | (uintptr_t)taps | (uintptr_t)bias | (uintptr_t)state) & 15) == 0;
        if (wide)
            conv_act8_kernel<<<(unsigned)((total / 8 + 255) / 256), 256, 0, stream>>>(
                (bf16_t*)out, (const bf16_t*)x, (const bf16_t*)taps, (const bf16_t*)bias, state, row_floats, tail_off, token_seq,
                cu_tokens, state_slots, C, k, x_ld, x_off, act, total / 8);
        else
        conv_act_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, (const bf16_t*)taps,
                                                            (const bf16_t*)bias, state, row_floats, tail_off, token_seq, cu_tokens,
                                                            state_slots, C, k, x_ld, x_off, act, total);
        if (k > 1)
            conv_tail_kernel<bf16_t><<<tail_grid, 256, 0, stream>>>(state, row_floats, tail_off, (const bf16_t*)x, cu_tokens,
                                                                    state_slots, C, k, x_ld, x_off);
    }
    IA_LAUNCH_CHECK("conv_act_step");
    return 0;
}

// ---- gates ----------------------------------------------------------------------------------------------------------
__device__ __forceinline__ float ls_softplus(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// Exponential gates under a running maximum, one thread a (request, head) over the request's tokens:
//     i = cap tanh((ri + bi) / cap),  f = logsigmoid(cap tanh((rf + bf) / cap)),  m_t = max(f + m_(t-1), i)
//     log_a = f + m_(t-1) - m_t,  b = exp(i - m_t),  floor = exp(-m_t)
// m starts at 0 and is kept in the state row.
template <typename T>
__global__ void exp_gates_kernel(float* __restrict__ log_a, float* __restrict__ b, float* __restrict__ floor_,
                                 float* __restrict__ state, long long row_floats, long long m_off,
                                 const T* __restrict__ proj, long long p_ld, int i_off, int f_off,
                                 const float* __restrict__ bias_i, const float* __restrict__ bias_f, float cap,
                                 const int* __restrict__ cu_tokens, const int* __restrict__ state_slots, int H, int n_seqs) {
    const int id = blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= n_seqs * H) return;
    const int seq = id / H, h = id - seq * H;
    float* mp = state + (long long)state_slots[seq] * row_floats + m_off + h;
    float m = *mp;
    const float bi = bias_i[h], bf = bias_f[h];
    for (int t = cu_tokens[seq]; t < cu_tokens[seq + 1]; ++t) {
        const float gi = cap * tanhf((ld(proj + (long long)t * p_ld + i_off + h) + bi) / cap);
        const float zf = cap * tanhf((ld(proj + (long long)t * p_ld + f_off + h) + bf) / cap);
        const float gf = -ls_softplus(-zf);
        const float m_new = fmaxf(gf + m, gi);
        log_a[(long long)t * H + h] = gf + m - m_new;
        b[(long long)t * H + h] = expf(gi - m_new);
        floor_[(long long)t * H + h] = expf(-m_new);
        m = m_new;
    }
    *mp = m;
}

// The same for long portions: a block a (request, head); thread i owns a run of neighbouring tokens.  A token's step
// m -> max(m + f, i) is the pair (f, i); two steps in a row are the pair (f1 + f2, max(i1 + f2, i2)), so the runs are
// folded first, the block's threads' pairs are folded in order by one thread, and every thread then walks its run from
// the maximum it starts with.  The sums of f inside a pair matter only while they are small (beyond that the second
// entry wins the maximum), so the result differs from the walk above by rounding only.
#define EG_THREADS 256
template <typename T>
__global__ __launch_bounds__(EG_THREADS) void exp_gates_block_kernel(
    float* __restrict__ log_a, float* __restrict__ b, float* __restrict__ floor_, float* __restrict__ state,
    long long row_floats, long long m_off, const T* __restrict__ proj, long long p_ld, int i_off, int f_off,
    const float* __restrict__ bias_i, const float* __restrict__ bias_f, float cap, const int* __restrict__ cu_tokens,
    const int* __restrict__ state_slots, int H) {
    __shared__ float sf[EG_THREADS], si[EG_THREADS], start[EG_THREADS];
    const int seq = blockIdx.x / H, h = blockIdx.x - seq * H;
    const int first = cu_tokens[seq], last = cu_tokens[seq + 1];
    const int per = (last - first + EG_THREADS - 1) / EG_THREADS;
    const int lo = first + threadIdx.x * per < last ? first + threadIdx.x * per : last;
    const int hi = lo + per < last ? lo + per : last;
    float* mp = state + (long long)state_slots[seq] * row_floats + m_off + h;
    const float bi = bias_i[h], bf = bias_f[h];
    // the run's gates (parked where the results go) and its pair
    float sum_f = 0.f, top = -INFINITY;
    for (int t = lo; t < hi; ++t) {
        const float gi = cap * tanhf((ld(proj + (long long)t * p_ld + i_off + h) + bi) / cap);
        const float zf = cap * tanhf((ld(proj + (long long)t * p_ld + f_off + h) + bf) / cap);
        const float gf = -ls_softplus(-zf);
        log_a[(long long)t * H + h] = gf;
        b[(long long)t * H + h] = gi;
        sum_f += gf;
        top = fmaxf(top + gf, gi);
    }
    sf[threadIdx.x] = sum_f; si[threadIdx.x] = top;
    __syncthreads();
    if (threadIdx.x == 0) {
        float m = *mp;
        for (int i = 0; i < EG_THREADS; ++i) {
            start[i] = m;
            m = fmaxf(m + sf[i], si[i]);                         // (an empty run is the pair (0, -inf): m stays)
        }
        *mp = m;
    }
    __syncthreads();
    float m = start[threadIdx.x];
    for (int t = lo; t < hi; ++t) {
        const float gf = log_a[(long long)t * H + h], gi = b[(long long)t * H + h];
        const float m_new = fmaxf(gf + m, gi);
        log_a[(long long)t * H + h] = gf + m - m_new;
        b[(long long)t * H + h] = expf(gi - m_new);
        floor_[(long long)t * H + h] = expf(-m_new);
        m = m_new;
    }
}

// max_q_len: an upper bound of the tokens a request brings (steps with long portions take a block a (request, head))
extern "C" int ia_exp_gates(float* log_a, float* b, float* floor_, float* state, long long row_floats, long long m_off,
                            const void* proj, long long p_ld, int i_off, int f_off, const float* bias_i,
                            const float* bias_f, float cap, const int* cu_tokens, const int* state_slots, int H,
                            int n_seqs, int max_q_len, int dtype, hipStream_t stream) {
    IA_CHECK(H > 0 && n_seqs >= 0 && cap > 0.f && i_off >= 0 && f_off >= 0 && i_off + H <= p_ld && f_off + H <= p_ld,
             "exp_gates: bad sizes heads=%d cap=%g", H, (double)cap);
    IA_CHECK(m_off >= 0 && m_off + H <= row_floats, "exp_gates: the maxima do not fit the state row");
    if (n_seqs == 0) return 0;
    if (max_q_len > 32) {
        if (dtype == IA_F32)
            exp_gates_block_kernel<float><<<(unsigned)(n_seqs * H), EG_THREADS, 0, stream>>>(
                log_a, b, floor_, state, row_floats, m_off, (const float*)proj, p_ld, i_off, f_off, bias_i, bias_f, cap, cu_tokens,
                state_slots, H);
        else
            exp_gates_block_kernel<bf16_t><<<(unsigned)(n_seqs * H), EG_THREADS, 0, stream>>>(
                log_a, b, floor_, state, row_floats, m_off, (const bf16_t*)proj, p_ld, i_off, f_off, bias_i, bias_f, cap, cu_tokens,
                state_slots, H);
        IA_LAUNCH_CHECK("exp_gates (blocks)");
        return 0;
    }
    const unsigned blocks = (unsigned)((n_seqs * H + 63) / 64);
    if (dtype == IA_F32)
        exp_gates_kernel<float><<<blocks, 64, 0, stream>>>(log_a, b, floor_, state, row_floats, m_off, (const float*)proj, p_ld,
                                                           i_off, f_off, bias_i, bias_f, cap, cu_tokens, state_slots, H, n_seqs);
    else
        exp_gates_kernel<bf16_t><<<blocks, 64, 0, stream>>>(log_a, b, floor_, state, row_floats, m_off, (const bf16_t*)proj, p_ld,
                                                            i_off, f_off, bias_i, bias_f, cap, cu_tokens, state_slots, H, n_seqs);
    IA_LAUNCH_CHECK("exp_gates");
    return 0;
}

// Step sizes of a selective state space, one thread a (token, head): dt = softplus(raw + bias),
// log_a = -exp(a_log) * dt, b = dt.
template <typename T>
__global__ void step_gates_kernel(float* __restrict__ log_a, float* __restrict__ b, const T* __restrict__ proj,
                                  long long p_ld, int dt_off, const float* __restrict__ dt_bias,
                                  const float* __restrict__ a_log, int H, long long total) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const long long t = i / H;
    const int h = (int)(i - t * H);
    const float dt = ls_softplus(ld(proj + t * p_ld + dt_off + h) + dt_bias[h]);
    log_a[i] = -expf(a_log[h]) * dt;
    b[i] = dt;
}

extern "C" int ia_step_gates(float* log_a, float* b, const void* proj, long long p_ld, int dt_off, const float* dt_bias,
                             const float* a_log, int n, int H, int dtype, hipStream_t stream) {
    IA_CHECK(n >= 0 && H > 0 && dt_off >= 0 && dt_off + H <= p_ld, "step_gates: bad sizes n=%d heads=%d", n, H);
    if (n == 0) return 0;
    const long long total = (long long)n * H;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (dtype == IA_F32)
        step_gates_kernel<float><<<blocks, 256, 0, stream>>>(log_a, b, (const float*)proj, p_ld, dt_off, dt_bias, a_log, H, total);
    else
        step_gates_kernel<bf16_t><<<blocks, 256, 0, stream>>>(log_a, b, (const bf16_t*)proj, p_ld, dt_off, dt_bias, a_log, H, total);
    IA_LAUNCH_CHECK("step_gates");
    return 0;
}

// ---- the recurrence ---------------------------------------------------------------------------------------------------
// A block owns a (request, head, tile of S's columns) and walks tokens in order.  A column j of S is shared by P
// neighbouring lanes, each with LS_R of the column's `dim` entries in registers; the lanes add up q . S[:, j] by a
// butterfly.  The operands of a stage of tokens (q, k, the block's columns of v, decays, input scales) come into shared
// memory together, already scaled, and the walk over the stage reads them from there.
//
// Three forms of one loop.  WALK: the request's tokens of this step from its state row and back into it (decode steps,
// short portions).  Long portions are cut into chunks of `chunk` tokens that run side by side: LOCAL walks a chunk from
// a state of zero, writes the chunk's outputs as if nothing came before it and leaves the chunk's final matrix and the
// product of its decays in a workspace; `chunk_states_kernel` then walks a request's chunks in order, S <- A_c S + U_c
// from the state row, leaving in the workspace the matrix each chunk starts from and in the state row the last one;
// CARRY adds to every output of a chunk what the matrix it started from contributes, (prod_(s<=t) a_s) S_c^T q_t.
// A token's result differs between the forms, and between chunk borders, by rounding only.
#define LS_R 8
#define LS_THREADS 256
enum { LS_WALK = 0, LS_LOCAL = 1, LS_CARRY = 2 };

struct ScanArgs {
    float* out;                 // [n][H][vdim]
    float* den;                 // [n][H]: the output of the column of ones, or null (no such column)
    float* state; long long row_floats, s_off;
    const void* q; long long q_ld; int q_off, q_heads;          // head h of H reads head h / (H / q_heads)
    const void* k; long long k_ld; int k_off, k_heads;
    const void* v; long long v_ld; int v_off;                    // [.., H, vdim]
    const float* log_a; int a_per_token;                          // logarithms of the decays [n][H]; with a_per_token 0 the decays themselves, [H]
    const float* b;                                               // [n][H] or null (1)
    const float* skip;                                            // [H] or null
    const int* cu_tokens; const int* state_slots;
    int H, dim, vdim, P, cols;                                    // cols: columns of S a block (LS_THREADS / P)
    float q_scale, k_scale;
    int wide;                                                     // the matrices' rows start at multiples of 16 bytes
    int q_vec, k_vec;                                             // so do the heads' rows of q and k, and dim is a multiple of a 16-byte load
    int stage;                                                    // tokens whose operands a block holds in shared memory at a time
    int chunk, max_chunks;                                        // LOCAL, CARRY: tokens of a chunk; chunks of the longest portion
    float* chunk_s;                                               // [seqs][max_chunks][H][vt][dim]
    float* chunk_a;                                               // [seqs][max_chunks][H]
};

template <typename T, int MODE, int P>
__global__ __launch_bounds__(LS_THREADS) void linear_scan_kernel(const ScanArgs a) {
    // a stage of tokens: q and k [stage][P * LS_R] (scaled, zeros beyond dim), the block's columns of v [stage][cols],
    // the decays and input scales [stage]
    extern __shared__ __attribute__((aligned(16))) float ls_stage[];
    constexpr int dimp = P * LS_R;                                // (P is a constant so that the butterfly runs on lane swaps)
    float* const q_s = ls_stage;
    float* const k_s = q_s + (size_t)a.stage * dimp;
    float* const v_s = k_s + (size_t)a.stage * dimp;
    float* const a_s = v_s + (size_t)a.stage * a.cols;
    float* const b_s = a_s + a.stage;
    const int p = threadIdx.x % P, jj = threadIdx.x / P;
    const int h = blockIdx.y;
    const int seq = MODE == LS_WALK ? blockIdx.z : blockIdx.z / a.max_chunks;
    const int c = MODE == LS_WALK ? 0 : blockIdx.z - seq * a.max_chunks;
    const int vt = a.vdim + (a.den != nullptr ? 1 : 0);           // columns of S
    const int j0 = blockIdx.x * a.cols, j = j0 + jj;
    const bool live = j < vt;
    const bool ones = j >= a.vdim;                                // the column whose value is always 1
    int first = a.cu_tokens[seq], last = a.cu_tokens[seq + 1];
    if (MODE != LS_WALK) {
        first += c * a.chunk;
        if (first >= last) return;                                // (the whole block: this request has fewer chunks)
        last = first + a.chunk < last ? first + a.chunk : last;
    }
    const int qh = h / (a.H / a.q_heads), kh = h / (a.H / a.k_heads);
    const int i0 = p * LS_R;
    const T* q = (const T*)a.q + a.q_off + (long long)qh * a.dim;
    const T* k = (const T*)a.k + a.k_off + (long long)kh * a.dim;
    const T* v = (const T*)a.v + a.v_off + (long long)h * a.vdim;
    const long long col = ((long long)h * vt + (live ? j : 0)) * a.dim + i0;
    float* srow = MODE == LS_WALK ? a.state + (long long)a.state_slots[seq] * a.row_floats + a.s_off + col
                                  : a.chunk_s + (long long)blockIdx.z * a.H * vt * a.dim + col;
    // (a thread's eight entries as two 16-byte accesses where the matrices' rows allow it: a decode step is this read
    // and the write at the end)
    const bool wide = a.wide && i0 + LS_R <= a.dim;
    float S[LS_R];
    if (MODE != LS_LOCAL && live && wide) {
        const float4 lo = *(const float4*)srow, hi = *(const float4*)(srow + 4);
        S[0] = lo.x; S[1] = lo.y; S[2] = lo.z; S[3] = lo.w; S[4] = hi.x; S[5] = hi.y; S[6] = hi.z; S[7] = hi.w;
    } else {
#pragma unroll
        for (int r = 0; r < LS_R; ++r) S[r] = (MODE != LS_LOCAL && live && i0 + r < a.dim) ? srow[r] : 0.f;
    }
    const float skip = a.skip != nullptr ? a.skip[h] : 0.f;
    float run = 1.f;                                              // the product of the decays so far
    for (int t0 = first; t0 < last; t0 += a.stage) {
        const int nt = last - t0 < a.stage ? last - t0 : a.stage;
        __syncthreads();                                          // (the stage before is used up)
        for (int e = threadIdx.x; e < nt * dimp; e += LS_THREADS) {
            const int tt = e / dimp, i = e - tt * dimp;
            q_s[e] = i < a.dim ? ld(q + (long long)(t0 + tt) * a.q_ld + i) * a.q_scale : 0.f;
            if (MODE != LS_CARRY) k_s[e] = i < a.dim ? ld(k + (long long)(t0 + tt) * a.k_ld + i) * a.k_scale : 0.f;
        }
        for (int e = threadIdx.x; e < nt * a.cols; e += LS_THREADS) {
            const int tt = e / a.cols, jv = j0 + e - tt * a.cols;
            if (MODE != LS_CARRY) v_s[e] = jv < a.vdim ? ld(v + (long long)(t0 + tt) * a.v_ld + jv) : 1.f;
            // (CARRY: what the chunk's own walk left at the places this block adds to, so that no load stands in the walk)
            else v_s[e] = jv < a.vdim ? a.out[((long long)(t0 + tt) * a.H + h) * a.vdim + jv]
                                      : jv < vt ? a.den[(long long)(t0 + tt) * a.H + h] : 0.f;
        }
        for (int e = threadIdx.x; e < nt; e += LS_THREADS) {
            const float an = a.log_a[a.a_per_token ? (long long)(t0 + e) * a.H + h : h];
            a_s[e] = a.a_per_token ? expf(an) : an;
            b_s[e] = a.b != nullptr ? a.b[(long long)(t0 + e) * a.H + h] : 1.f;
        }
        __syncthreads();
#pragma unroll 2
        for (int tt = 0; tt < nt; ++tt) {
            const float4 qa = *(const float4*)(q_s + tt * dimp + i0), qb = *(const float4*)(q_s + tt * dimp + i0 + 4);
            const float qc[LS_R] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
            const float decay = a_s[tt];
            run *= decay;
            float part = 0.f, vc = 0.f;
            if (MODE != LS_CARRY) {
                const float4 ka = *(const float4*)(k_s + tt * dimp + i0), kb = *(const float4*)(k_s + tt * dimp + i0 + 4);
                const float kc[LS_R] = {ka.x, ka.y, ka.z, ka.w, kb.x, kb.y, kb.z, kb.w};
                vc = v_s[tt * a.cols + jj];
                const float bv = b_s[tt] * vc;
#pragma unroll
                for (int r = 0; r < LS_R; ++r) S[r] = fmaf(decay, S[r], bv * kc[r]);
            }
#pragma unroll
            for (int r = 0; r < LS_R; ++r) part = fmaf(S[r], qc[r], part);
#pragma unroll
            for (int o = P / 2; o > 0; o >>= 1) part += __shfl_xor(part, o, IA_WAVE);
            if (p == 0 && live) {
                const int t = t0 + tt;
                float* at = ones ? a.den + (long long)t * a.H + h : a.out + ((long long)t * a.H + h) * a.vdim + j;
                if (MODE == LS_CARRY) *at = fmaf(run, part, v_s[tt * a.cols + jj]);
                else *at = ones ? part : fmaf(skip, vc, part);
            }
        }
    }
    if (MODE == LS_CARRY) return;
    if (live && wide) {
        *(float4*)srow = make_float4(S[0], S[1], S[2], S[3]);
        *(float4*)(srow + 4) = make_float4(S[4], S[5], S[6], S[7]);
    } else if (live) {
#pragma unroll
        for (int r = 0; r < LS_R; ++r)
            if (i0 + r < a.dim) srow[r] = S[r];
    }
    if (MODE == LS_LOCAL && blockIdx.x == 0 && threadIdx.x == 0) a.chunk_a[(long long)blockIdx.z * a.H + h] = run;
}

// CARRY on the matrix cores in their true 32-bit form (`v_mfma_f32_16x16x4_f32`: 32-bit operands, products and sums),
// for keys of up to 128 entries and chunks of up to 64 tokens: a chunk's share of its start is a product of its queries
// [tokens x dim] with the matrix it starts from [dim x columns], row t scaled by the product of the decays up to t.  A
// block of four waves owns a (chunk, head, 32 columns); the queries (scaled) and the columns come into shared memory
// once, rows `ld` floats apart; wave w owns tokens 16 w .. 16 w + 15.  Lane l supplies A[l % 16][l / 16] and
// B[l / 16][l % 16] of a step of four k and receives D[4 (l / 16) + r][l % 16].
typedef float ls_f32x4 __attribute__((ext_vector_type(4)));
#define LC_TOKENS 64

// Rows of a chunk into shared memory as 32-bit values times `scale`: dst[tt][i] = src[(first + tt) * src_ld + i] for tt <
// nt and i < dim, zeros up to 64 rows and k4 columns.  `vec`: 16-byte loads (the rows start at multiples of 16 bytes and
// dim is a multiple of what a load holds); every load of a thread is asked for before its first store.
__device__ __forceinline__ void ls_load16(const float* p, float (&v)[8], int& n) {
    const float4 q = *(const float4*)p;
    v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w; n = 4;
}
__device__ __forceinline__ void ls_load16(const bf16_t* p, float (&v)[8], int& n) { ls_unpack8(p, v); n = 8; }

template <typename T>
__device__ __forceinline__ void stage_rows(float* __restrict__ dst, int ld_s, const T* __restrict__ src, long long src_ld,
                                           int first, int nt, int dim, int k4, float scale, bool vec) {
    constexpr int E = 16 / (int)sizeof(T);                // elements a load
    if (vec) {
        const int per_row = dim / E;                       // (k4 == dim here)
        const int total = LC_TOKENS * per_row;             // at most 64 * 32 = 8 rounds of the block
        float v[8][8];
        int n = E;
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            const int idx = threadIdx.x + 256 * it;
            const int tt = idx / per_row, piece = idx - tt * per_row;
            if (idx < total && tt < nt) ls_load16(src + (long long)(first + tt) * src_ld + piece * E, v[it], n);
            else {
#pragma unroll
                for (int e = 0; e < 8; ++e) v[it][e] = 0.f;
            }
        }
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            const int idx = threadIdx.x + 256 * it;
            const int tt = idx / per_row, piece = idx - tt * per_row;
            if (idx < total) {
#pragma unroll
                for (int e = 0; e < E; ++e) dst[tt * ld_s + piece * E + e] = v[it][e] * scale;
            }
        }
        return;
    }
    // element by element: 8 rows x 4 columns a thread (k4 <= 128), the loads first
    float v[8][4];
#pragma unroll
    for (int it = 0; it < 8; ++it)
#pragma unroll
        for (int ic = 0; ic < 4; ++ic) {
            const int tt = (threadIdx.x >> 5) + 8 * it, i = (threadIdx.x & 31) + 32 * ic;
            v[it][ic] = (tt < nt && i < dim) ? ld(src + (long long)(first + tt) * src_ld + i) : 0.f;
        }
#pragma unroll
    for (int it = 0; it < 8; ++it)
#pragma unroll
        for (int ic = 0; ic < 4; ++ic) {
            const int tt = (threadIdx.x >> 5) + 8 * it, i = (threadIdx.x & 31) + 32 * ic;
            if (i < k4) dst[tt * ld_s + i] = v[it][ic] * scale;
        }
}
#define LC_COLS 32
#define LC_MAX_DIM 128

template <typename T>
__global__ __launch_bounds__(256) void linear_carry_mfma_kernel(const ScanArgs a, int ld_s) {
    extern __shared__ __attribute__((aligned(16))) float lc_shared[];
    float* const q_s = lc_shared;                          // [LC_TOKENS][ld_s]
    float* const s_s = q_s + LC_TOKENS * ld_s;             // [LC_COLS][ld_s]
    float* const run_s = s_s + LC_COLS * ld_s;             // [LC_TOKENS]
    const int h = blockIdx.y;
    const int seq = blockIdx.z / a.max_chunks, c = blockIdx.z - seq * a.max_chunks;
    const int vt = a.vdim + (a.den != nullptr ? 1 : 0);
    const int j0 = blockIdx.x * LC_COLS;
    const int first = a.cu_tokens[seq] + c * a.chunk, end = a.cu_tokens[seq + 1];
    if (first >= end) return;                              // (the whole block)
    const int nt = end - first < a.chunk ? end - first : a.chunk;
    const int k4 = (a.dim + 3) / 4 * 4;
    const T* q = (const T*)a.q + a.q_off + (long long)(h / (a.H / a.q_heads)) * a.dim;
    stage_rows<T>(q_s, ld_s, q, a.q_ld, first, nt, a.dim, k4, a.q_scale, a.q_vec != 0);
    // (the columns of the start's matrix lie like rows of dim entries: the same staging, 32 of them)
    const float* start = a.chunk_s + ((long long)blockIdx.z * a.H + h) * vt * a.dim;
    const int cols_here = vt - j0 < LC_COLS ? vt - j0 : LC_COLS;
    if (a.wide) {
        const int per_row = a.dim / 4;
        for (int idx = threadIdx.x; idx < LC_COLS * per_row; idx += 256) {
            const int jj = idx / per_row, piece = idx - jj * per_row;
            const float4 z = jj < cols_here ? *(const float4*)(start + (long long)(j0 + jj) * a.dim + 4 * piece) : make_float4(0.f, 0.f, 0.f, 0.f);
            *(float4*)(s_s + jj * ld_s + 4 * piece) = z;
        }
    } else {
        for (int e = threadIdx.x; e < LC_COLS * k4; e += 256) {
            const int jj = e / k4, i = e - jj * k4;
            s_s[jj * ld_s + i] = (jj < cols_here && i < a.dim) ? start[(long long)(j0 + jj) * a.dim + i] : 0.f;
        }
    }
    if (threadIdx.x < LC_TOKENS) {
        // the products of the decays up to each token: the first wave's lanes load one decay each and fold them by lane shifts
        const int tt = threadIdx.x;
        float run = 1.f;
        if (tt < nt) {
            const float an = a.log_a[a.a_per_token ? (long long)(first + tt) * a.H + h : h];
            run = a.a_per_token ? expf(an) : an;
        }
#pragma unroll
        for (int o = 1; o < LC_TOKENS; o <<= 1) {
            const float before = __shfl_up(run, o, IA_WAVE);
            if (tt >= o) run *= before;
        }
        run_s[tt] = run;
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, kq = lane >> 4;
    ls_f32x4 acc[LC_COLS / 16];
#pragma unroll
    for (int ct = 0; ct < LC_COLS / 16; ++ct) acc[ct] = (ls_f32x4){0.f, 0.f, 0.f, 0.f};
    const float* qa = q_s + (16 * wave + r16) * ld_s + kq;
    const float* sb = s_s + r16 * ld_s + kq;
    for (int k0 = 0; k0 < k4; k0 += 4) {
        const float av = qa[k0];
#pragma unroll
        for (int ct = 0; ct < LC_COLS / 16; ++ct)
            acc[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, sb[16 * ct * ld_s + k0], acc[ct], 0, 0, 0);
    }
#pragma unroll
    for (int ct = 0; ct < LC_COLS / 16; ++ct) {
        const int col = j0 + 16 * ct + r16;
        if (col >= vt) continue;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int tt = 16 * wave + 4 * kq + r;
            if (tt >= nt) continue;
            const long long t = first + tt;
            float* at = col < a.vdim ? a.out + (t * a.H + h) * a.vdim + col : a.den + t * a.H + h;
            *at = fmaf(run_s[tt], acc[ct][r], *at);
        }
    }
}

// LOCAL on the same instruction, for the same sizes: a block of four waves owns a (chunk, head).  With G_t the sum of
// the decays' logarithms up to t (inclusive) and b_s the input scales,
//     P[t][s] = (q_t . k_s) exp(G_t - G_s) b_s  for s <= t (0 beyond),      out_t = sum_s P[t][s] v_s (+ skip v_t),
//     U = sum_s exp(G_last - G_s) b_s k_s v_s^T,                             A = exp(G_last).
// The queries and keys of the chunk (scaled, zeros for tokens it does not have) come into shared memory once; the
// scores are formed once and weighted, then the columns of v come 32 at a time: a product with P for the outputs, a
// product with the weighted keys for the chunk's matrix.  Every exponent is <= 0.  A decay of 0 has the logarithm
// -1e4, so that differences stay numbers.  Wave w owns tokens 16 w .. 16 w + 15 of the outputs and rows 16 w .., 16 (w +
// 4) .. of the chunk's matrix.
#define LL_P_LD 68
#define LL_V_LD 36

template <typename T>
__global__ __launch_bounds__(256) void linear_local_mfma_kernel(const ScanArgs a, int ld_s) {
    extern __shared__ __attribute__((aligned(16))) float ll_shared[];
    // (The scores take the place of the queries where a row of queries is long enough for a row of scores: a wave
    // writes the scores of its 16 tokens after it has read those tokens' queries, and nobody else reads them.  Two
    // blocks then fit a compute unit's shared memory at keys of 128.)
    const bool over = ld_s >= LL_P_LD;
    const int p_ld = over ? ld_s : LL_P_LD;
    float* const q_s = ll_shared;                          // [64][ld_s]
    float* const k_s = q_s + LC_TOKENS * ld_s;             // [64][ld_s]
    float* const p_s = over ? q_s : k_s + LC_TOKENS * ld_s;   // [64][p_ld]
    float* const v_s = k_s + LC_TOKENS * ld_s + (over ? 0 : LC_TOKENS * LL_P_LD);   // [64][LL_V_LD]
    float* const g_s = v_s + LC_TOKENS * LL_V_LD;          // [64] G_t
    float* const b_s = g_s + LC_TOKENS;                    // [64] b_s
    float* const w_s = b_s + LC_TOKENS;                    // [64] exp(G_last - G_s) b_s
    const int h = blockIdx.y;
    const int seq = blockIdx.z / a.max_chunks, c = blockIdx.z - seq * a.max_chunks;
    const int vt = a.vdim + (a.den != nullptr ? 1 : 0);
    const int first = a.cu_tokens[seq] + c * a.chunk, end = a.cu_tokens[seq + 1];
    if (first >= end) return;                              // (the whole block)
    const int nt = end - first < a.chunk ? end - first : a.chunk;
    const int k4 = (a.dim + 3) / 4 * 4;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, kq = lane >> 4;
    const T* q = (const T*)a.q + a.q_off + (long long)(h / (a.H / a.q_heads)) * a.dim;
    const T* k = (const T*)a.k + a.k_off + (long long)(h / (a.H / a.k_heads)) * a.dim;
    const T* v = (const T*)a.v + a.v_off + (long long)h * a.vdim;
    stage_rows<T>(q_s, ld_s, q, a.q_ld, first, nt, a.dim, k4, a.q_scale, a.q_vec != 0);
    stage_rows<T>(k_s, ld_s, k, a.k_ld, first, nt, a.dim, k4, a.k_scale, a.k_vec != 0);
    if (threadIdx.x < LC_TOKENS) {
        const int tt = threadIdx.x;
        float g = 0.f, b = 0.f;
        if (tt < nt) {
            const float an = a.log_a[a.a_per_token ? (long long)(first + tt) * a.H + h : h];
            g = fmaxf(a.a_per_token ? an : logf(an), -1e4f);
            b = a.b != nullptr ? a.b[(long long)(first + tt) * a.H + h] : 1.f;
        }
#pragma unroll
        for (int o = 1; o < LC_TOKENS; o <<= 1) {
            const float before = __shfl_up(g, o, IA_WAVE);
            if (tt >= o) g += before;
        }
        const float g_last = __shfl(g, LC_TOKENS - 1, IA_WAVE);
        g_s[tt] = g; b_s[tt] = b; w_s[tt] = expf(g_last - g) * b;
        if (tt == 0) a.chunk_a[(long long)blockIdx.z * a.H + h] = expf(g_last);
    }
    __syncthreads();
    // ---- the weighted scores ------------------------------------------------------------------------------------
    {
        ls_f32x4 acc[4];
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) acc[ct] = (ls_f32x4){0.f, 0.f, 0.f, 0.f};
        const float* qa = q_s + (16 * wave + r16) * ld_s + kq;
        const float* kb = k_s + r16 * ld_s + kq;
        for (int k0 = 0; k0 < k4; k0 += 4) {
            const float av = qa[k0];
#pragma unroll
            for (int ct = 0; ct < 4; ++ct)
                acc[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, kb[16 * ct * ld_s + k0], acc[ct], 0, 0, 0);
        }
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
            const int s = 16 * ct + r16;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int t = 16 * wave + 4 * kq + r;
                p_s[t * p_ld + s] = s <= t ? acc[ct][r] * expf(g_s[t] - g_s[s]) * b_s[s] : 0.f;
            }
        }
    }
    const float skip = a.skip != nullptr ? a.skip[h] : 0.f;
    float* const u_out = a.chunk_s + ((long long)blockIdx.z * a.H + h) * vt * a.dim;
    const int row_tiles = (a.dim + 15) / 16;
    for (int j0 = 0; j0 < vt; j0 += 32) {
        __syncthreads();                                   // (the scores are written; the columns before are used up)
        {
            const int j = j0 + (threadIdx.x & 31);
            float vv[8];
#pragma unroll
            for (int it = 0; it < 8; ++it) {
                const int tt = (threadIdx.x >> 5) + 8 * it;
                vv[it] = (tt < nt && j < vt) ? (j < a.vdim ? ld(v + (long long)(first + tt) * a.v_ld + j) : 1.f) : 0.f;
            }
#pragma unroll
            for (int it = 0; it < 8; ++it) v_s[((threadIdx.x >> 5) + 8 * it) * LL_V_LD + (threadIdx.x & 31)] = vv[it];
        }
        __syncthreads();
        // the outputs of the chunk's own tokens
        {
            ls_f32x4 acc[2] = {(ls_f32x4){0.f, 0.f, 0.f, 0.f}, (ls_f32x4){0.f, 0.f, 0.f, 0.f}};
            const float* pa = p_s + (16 * wave + r16) * p_ld + kq;
            const float* vb = v_s + kq * LL_V_LD + r16;
#pragma unroll 4
            for (int k0 = 0; k0 < LC_TOKENS; k0 += 4) {
                const float av = pa[k0];
                acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, vb[k0 * LL_V_LD], acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, vb[k0 * LL_V_LD + 16], acc[1], 0, 0, 0);
            }
#pragma unroll
            for (int c2 = 0; c2 < 2; ++c2) {
                const int col = j0 + 16 * c2 + r16;
                if (col >= vt) continue;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int tt = 16 * wave + 4 * kq + r;
                    if (tt >= nt) continue;
                    const long long t = first + tt;
                    if (col < a.vdim) a.out[(t * a.H + h) * a.vdim + col] = fmaf(skip, v_s[tt * LL_V_LD + 16 * c2 + r16], acc[c2][r]);
                    else a.den[t * a.H + h] = acc[c2][r];
                }
            }
        }
        // the chunk's matrix: rows 16 mt .. of U against these columns
        for (int mt = wave; mt < row_tiles; mt += 4) {
            ls_f32x4 acc[2] = {(ls_f32x4){0.f, 0.f, 0.f, 0.f}, (ls_f32x4){0.f, 0.f, 0.f, 0.f}};
            const float* ka = k_s + kq * ld_s + 16 * mt + r16;
            const float* vb = v_s + kq * LL_V_LD + r16;
#pragma unroll 4
            for (int k0 = 0; k0 < LC_TOKENS; k0 += 4) {
                const float av = ka[k0 * ld_s] * w_s[k0 + kq];
                acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, vb[k0 * LL_V_LD], acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, vb[k0 * LL_V_LD + 16], acc[1], 0, 0, 0);
            }
#pragma unroll
            for (int c2 = 0; c2 < 2; ++c2) {
                const int col = j0 + 16 * c2 + r16;
                if (col >= vt) continue;
                const int i = 16 * mt + 4 * kq;
                float* at = u_out + (long long)col * a.dim + i;
                if (a.wide && i + 4 <= a.dim) *(float4*)at = make_float4(acc[c2][0], acc[c2][1], acc[c2][2], acc[c2][3]);
                else {
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (i + r < a.dim) at[r] = acc[c2][r];
                }
            }
        }
    }
}

// A request's chunks in order, one thread an entry of the heads' matrices: the workspace's U_c becomes the matrix that
// chunk c starts from, the state row takes the matrix behind the last chunk.
__global__ void chunk_states_kernel(float* __restrict__ chunk_s, const float* __restrict__ chunk_a, float* __restrict__ state,
                                    long long row_floats, long long s_off, const int* __restrict__ cu_tokens,
                                    const int* __restrict__ state_slots, int per_head, int H, int chunk, int max_chunks) {
    const long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long per_seq = (long long)H * per_head;
    if (e >= per_seq) return;
    const int seq = blockIdx.y;
    const int h = (int)(e / per_head);
    const int n_tokens = cu_tokens[seq + 1] - cu_tokens[seq];
    const int chunks = (n_tokens + chunk - 1) / chunk;
    float* srow = state + (long long)state_slots[seq] * row_floats + s_off + e;
    float S = *srow;
    for (int c = 0; c < chunks; ++c) {
        const long long unit = (long long)seq * max_chunks + c;
        float* u = chunk_s + unit * per_seq + e;
        const float mine = *u;
        *u = S;
        S = fmaf(chunk_a[unit * H + h], S, mine);
    }
    *srow = S;
}

// (tests switch the matrix cores' form of CARRY off to compare it with the vector units')
static int g_carry_mfma = 1;
extern "C" void ia_linear_scan_tune(int carry_mfma) { g_carry_mfma = carry_mfma; }

extern "C" long long ia_linear_scan_workspace(int n_seqs, int max_q_len, int chunk, int H, int dim, int vdim, int normaliser) {
    if (chunk <= 0 || n_seqs <= 0) return 0;
    const long long max_chunks = (max_q_len + chunk - 1) / chunk;
    return (long long)n_seqs * max_chunks * ((long long)H * (vdim + (normaliser ? 1 : 0)) * dim + H);
}

// chunk 0: every request's tokens are walked from its state row.  chunk > 0: portions are cut into chunks of that many
// tokens that run side by side; `workspace` holds ia_linear_scan_workspace(...) floats and max_q_len is an upper bound
// of the tokens a request brings.
extern "C" int ia_linear_scan(float* out, float* den, float* state, long long row_floats, long long s_off,
                              const void* q, long long q_ld, int q_off, int q_heads,
                              const void* k, long long k_ld, int k_off, int k_heads,
                              const void* v, long long v_ld, int v_off,
                              const float* log_a, int a_per_token, const float* b, const float* skip,
                              const int* cu_tokens, const int* state_slots, int n_seqs, int H, int dim, int vdim,
                              float q_scale, float k_scale, int chunk, int max_q_len, float* workspace, int dtype,
                              hipStream_t stream) {
    IA_CHECK(n_seqs >= 0 && H > 0 && dim > 0 && vdim > 0, "linear_scan: bad sizes heads=%d dim=%d vdim=%d", H, dim, vdim);
    IA_CHECK(dim <= LS_R * IA_WAVE, "linear_scan: a key size of %d is beyond %d", dim, LS_R * IA_WAVE);
    IA_CHECK(q_heads > 0 && k_heads > 0 && H % q_heads == 0 && H % k_heads == 0,
             "linear_scan: %d heads over %d query and %d key heads", H, q_heads, k_heads);
    const int vt = vdim + (den != nullptr ? 1 : 0);
    IA_CHECK(s_off >= 0 && s_off + (long long)H * vt * dim <= row_floats, "linear_scan: the matrices do not fit the state row");
    IA_CHECK(q_off >= 0 && q_off + (long long)q_heads * dim <= q_ld && k_off >= 0 && k_off + (long long)k_heads * dim <= k_ld &&
             v_off >= 0 && v_off + (long long)H * vdim <= v_ld, "linear_scan: q, k or v lie outside their rows");
    IA_CHECK(chunk >= 0 && (chunk == 0 || (workspace != nullptr && max_q_len >= 1)), "linear_scan: chunks of %d tokens need a "
             "workspace and the longest portion's length", chunk);
    if (n_seqs == 0) return 0;
    int P = 1;
    while (P * LS_R < dim) P *= 2;
    ScanArgs a;
    a.out = out; a.den = den; a.state = state; a.row_floats = row_floats; a.s_off = s_off;
    a.q = q; a.q_ld = q_ld; a.q_off = q_off; a.q_heads = q_heads;
    a.k = k; a.k_ld = k_ld; a.k_off = k_off; a.k_heads = k_heads;
    a.v = v; a.v_ld = v_ld; a.v_off = v_off;
    a.log_a = log_a; a.a_per_token = a_per_token; a.b = b; a.skip = skip;
    a.cu_tokens = cu_tokens; a.state_slots = state_slots;
    a.H = H; a.dim = dim; a.vdim = vdim; a.P = P; a.cols = LS_THREADS / P;
    a.q_scale = q_scale; a.k_scale = k_scale;
    a.chunk = chunk; a.max_chunks = chunk ? (max_q_len + chunk - 1) / chunk : 1;
    a.chunk_s = workspace;
    {
        const int per = dtype == IA_F32 ? 4 : 8;                  // elements a 16-byte load
        a.q_vec = dim % per == 0 && q_off % per == 0 && q_ld % per == 0 && ((uintptr_t)q & 15) == 0;
        a.k_vec = dim % per == 0 && k_off % per == 0 && k_ld % per == 0 && ((uintptr_t)k & 15) == 0;
    }
    a.wide = dim % 4 == 0 && s_off % 4 == 0 && row_floats % 4 == 0 && ((uintptr_t)state & 15) == 0 && ((uintptr_t)workspace & 15) == 0;
    a.chunk_a = workspace ? workspace + (long long)n_seqs * a.max_chunks * H * vt * dim : nullptr;
    IA_CHECK((long long)n_seqs * a.max_chunks <= 65535, "linear_scan: %d requests x %d chunks exceed the grid", n_seqs, a.max_chunks);
    const unsigned tiles = (unsigned)((vt + a.cols - 1) / a.cols);
    // a stage: as many tokens as 32 KB of shared memory hold (2 to 32), no more than a walk can have
    const int per_token = 2 * P * LS_R + a.cols + 2;
    int stage = 32 * 1024 / 4 / per_token;
    stage = stage > 32 ? 32 : stage < 2 ? 2 : stage;
    const int longest = chunk ? chunk : (max_q_len >= 1 ? max_q_len : 1);
    a.stage = stage < longest ? stage : longest;
    const size_t shm = (size_t)a.stage * per_token * sizeof(float);
#define LS_LAUNCH_P(MODE, GRID, PP)                                                                            \
    do {                                                                                                       \
        if (dtype == IA_F32) linear_scan_kernel<float, MODE, PP><<<GRID, LS_THREADS, shm, stream>>>(a);        \
        else linear_scan_kernel<bf16_t, MODE, PP><<<GRID, LS_THREADS, shm, stream>>>(a);                       \
    } while (0)
#define LS_LAUNCH(MODE, GRID)                                                                                  \
    do {                                                                                                       \
        switch (P) {                                                                                           \
            case 1: LS_LAUNCH_P(MODE, GRID, 1); break;                                                         \
            case 2: LS_LAUNCH_P(MODE, GRID, 2); break;                                                         \
            case 4: LS_LAUNCH_P(MODE, GRID, 4); break;                                                         \
            case 8: LS_LAUNCH_P(MODE, GRID, 8); break;                                                         \
            case 16: LS_LAUNCH_P(MODE, GRID, 16); break;                                                       \
            case 32: LS_LAUNCH_P(MODE, GRID, 32); break;                                                       \
            default: LS_LAUNCH_P(MODE, GRID, 64); break;                                                       \
        }                                                                                                      \
    } while (0)
    if (chunk == 0) {
        const dim3 grid(tiles, (unsigned)H, (unsigned)n_seqs);
        LS_LAUNCH(LS_WALK, grid);
        IA_LAUNCH_CHECK("linear_scan");
        return 0;
    }
    const dim3 grid(tiles, (unsigned)H, (unsigned)(n_seqs * a.max_chunks));
    const int per_head = vt * dim;
    const dim3 sgrid((unsigned)(((long long)H * per_head + 255) / 256), (unsigned)n_seqs);
    const bool cores = g_carry_mfma && dim <= LC_MAX_DIM && chunk <= LC_TOKENS;
    if (cores) {
        const int ld_s = (dim + 3) / 4 * 4 + 4;
        const dim3 lgrid(1, (unsigned)H, (unsigned)(n_seqs * a.max_chunks));
        const int lshm = (int)((2 * LC_TOKENS * ld_s + LC_TOKENS * ((ld_s >= LL_P_LD ? 0 : LL_P_LD) + LL_V_LD) + 3 * LC_TOKENS) * sizeof(float));
        static int asked_f32 = 0, asked_bf16 = 0;          // shared memory beyond 64 KiB has to be asked for, once per instantiation
        int& asked = dtype == IA_F32 ? asked_f32 : asked_bf16;
        if (lshm > asked) {
            const hipError_t e = dtype == IA_F32
                ? hipFuncSetAttribute((const void*)linear_local_mfma_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, 112 * 1024)
                : hipFuncSetAttribute((const void*)linear_local_mfma_kernel<bf16_t>, hipFuncAttributeMaxDynamicSharedMemorySize, 112 * 1024);
            IA_CHECK(e == hipSuccess, "linear_scan: cannot ask for %d bytes of shared memory: %s", 112 * 1024, hipGetErrorString(e));
            asked = 112 * 1024;
        }
        if (dtype == IA_F32) linear_local_mfma_kernel<float><<<lgrid, 256, lshm, stream>>>(a, ld_s);
        else linear_local_mfma_kernel<bf16_t><<<lgrid, 256, lshm, stream>>>(a, ld_s);
    } else {
        LS_LAUNCH(LS_LOCAL, grid);
    }
    chunk_states_kernel<<<sgrid, 256, 0, stream>>>(a.chunk_s, a.chunk_a, state, row_floats, s_off, cu_tokens, state_slots, per_head,
                                                   H, chunk, a.max_chunks);
    if (cores) {
        const int ld_s = (dim + 3) / 4 * 4 + 4;
        const dim3 cgrid((unsigned)((vt + LC_COLS - 1) / LC_COLS), (unsigned)H, (unsigned)(n_seqs * a.max_chunks));
        const size_t cshm = (size_t)((LC_TOKENS + LC_COLS) * ld_s + LC_TOKENS) * sizeof(float);
        if (dtype == IA_F32) linear_carry_mfma_kernel<float><<<cgrid, 256, cshm, stream>>>(a, ld_s);
        else linear_carry_mfma_kernel<bf16_t><<<cgrid, 256, cshm, stream>>>(a, ld_s);
    } else {
        LS_LAUNCH(LS_CARRY, grid);
    }
#undef LS_LAUNCH
#undef LS_LAUNCH_P
    IA_LAUNCH_CHECK("linear_scan (chunks)");
    return 0;
}

// ---- what follows the recurrence: a norm a group of features, a gate, an optional division --------------------------
//     y = o / (max(|den|, floor) + 1e-6)        (with den: the matrix memory's normaliser, a (token, head))
//     y = y * act(g)                            (gate_first: gated, then normed)
//     y = y / rms(y over its group) * w         (groups of `group` neighbouring features; w may be null)
//     y = y * act(g)                            (otherwise the gate comes behind it)
// One wave a (token, group); 32-bit throughout, rounded once when it is stored.  act: 1 SiLU, 4 sigmoid.
__device__ __forceinline__ float ls_gate(float g, int act) {
    const float s = 1.0f / (1.0f + expf(-g));
    return act == IA_ACT_SILU ? g * s : s;
}

template <typename T>
__global__ __launch_bounds__(256) void group_norm_gate_kernel(
    T* __restrict__ out, const float* __restrict__ o, const float* __restrict__ den, const float* __restrict__ floor_,
    int head, const T* __restrict__ gate, long long g_ld, int g_off, int act, int gate_first,
    const float* __restrict__ w, float eps, int inner, int group, long long units) {
    const long long unit = (long long)blockIdx.x * (blockDim.x / IA_WAVE) + threadIdx.x / IA_WAVE;
    if (unit >= units) return;
    const int lane = threadIdx.x & (IA_WAVE - 1);
    const int per_row = inner / group;
    const long long t = unit / per_row;
    const int c0 = (int)(unit - t * per_row) * group;
    const int H = inner / head;
    auto value = [&](int c) {
        float y = o[t * inner + c];
        if (den != nullptr) {
            const long long at = t * H + c / head;
            y = y / (fmaxf(fabsf(den[at]), floor_[at]) + 1e-6f);
        }
        if (gate != nullptr && gate_first) y *= ls_gate(ld(gate + t * g_ld + g_off + c), act);
        return y;
    };
    float sq = 0.f;
    for (int c = c0 + lane; c < c0 + group; c += IA_WAVE) {
        const float y = value(c);
        sq = fmaf(y, y, sq);
    }
    const float rs = 1.0f / sqrtf(wave_sum(sq) / (float)group + eps);
    for (int c = c0 + lane; c < c0 + group; c += IA_WAVE) {
        float y = value(c) * rs;
        if (w != nullptr) y *= w[c];
        if (gate != nullptr && !gate_first) y *= ls_gate(ld(gate + t * g_ld + g_off + c), act);
        st(out + t * inner + c, y);
    }
}

// The same with a block a (token, group), for groups of many features.
template <typename T>
__global__ __launch_bounds__(1024) void group_norm_gate_block_kernel(
    T* __restrict__ out, const float* __restrict__ o, const float* __restrict__ den, const float* __restrict__ floor_,
    int head, const T* __restrict__ gate, long long g_ld, int g_off, int act, int gate_first,
    const float* __restrict__ w, float eps, int inner, int group) {
    __shared__ float scratch[16];
    const int per_row = inner / group;
    const long long t = blockIdx.x / per_row;
    const int c0 = (int)(blockIdx.x - t * per_row) * group;
    const int H = inner / head;
    auto value = [&](int c) {
        float y = o[t * inner + c];
        if (den != nullptr) {
            const long long at = t * H + c / head;
            y = y / (fmaxf(fabsf(den[at]), floor_[at]) + 1e-6f);
        }
        if (gate != nullptr && gate_first) y *= ls_gate(ld(gate + t * g_ld + g_off + c), act);
        return y;
    };
    float sq = 0.f;
    for (int c = c0 + threadIdx.x; c < c0 + group; c += blockDim.x) {
        const float y = value(c);
        sq = fmaf(y, y, sq);
    }
    const float rs = 1.0f / sqrtf(block_sum(sq, scratch) / (float)group + eps);
    for (int c = c0 + threadIdx.x; c < c0 + group; c += blockDim.x) {
        float y = value(c) * rs;
        if (w != nullptr) y *= w[c];
        if (gate != nullptr && !gate_first) y *= ls_gate(ld(gate + t * g_ld + g_off + c), act);
        st(out + t * inner + c, y);
    }
}

extern "C" int ia_group_norm_gate(void* out, const float* o, const float* den, const float* floor_, int head,
                                  const void* gate, long long g_ld, int g_off, int act, int gate_first, const float* w,
                                  float eps, int n, int inner, int group, int dtype, hipStream_t stream) {
    IA_CHECK(n >= 0 && inner > 0 && group > 0 && inner % group == 0 && head > 0 && inner % head == 0,
             "group_norm_gate: %d features in groups of %d, heads of %d", inner, group, head);
    IA_CHECK((den == nullptr) == (floor_ == nullptr), "group_norm_gate: a normaliser and its floor come together");
    IA_CHECK(gate == nullptr || ((act == IA_ACT_SILU || act == 4) && g_off >= 0 && g_off + inner <= g_ld),
             "group_norm_gate: gate activation %d (1 SiLU, 4 sigmoid) at %d of %lld", act, g_off, g_ld);
    if (n == 0) return 0;
    const long long units = (long long)n * (inner / group);
    IA_CHECK(units < 2147483647LL, "group_norm_gate: %d tokens x %d groups exceed the grid", n, inner / group);
    if (group > 256) {
        // (four features a thread where the group is wide enough: steps of few tokens have few blocks, and a block's
        // walk over its group is what they wait for)
        const int threads = group >= 4096 ? 1024 : group >= 2048 ? 512 : 256;
        if (dtype == IA_F32)
            group_norm_gate_block_kernel<float><<<(unsigned)units, threads, 0, stream>>>((float*)out, o, den, floor_, head, (const float*)gate,
                                                                                  g_ld, g_off, act, gate_first, w, eps, inner, group);
        else
            group_norm_gate_block_kernel<bf16_t><<<(unsigned)units, threads, 0, stream>>>((bf16_t*)out, o, den, floor_, head,
                                                                                   (const bf16_t*)gate, g_ld, g_off, act, gate_first, w,
                                                                                   eps, inner, group);
        IA_LAUNCH_CHECK("group_norm_gate (blocks)");
        return 0;
    }
    const unsigned blocks = (unsigned)((units + 3) / 4);
    if (dtype == IA_F32)
        group_norm_gate_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, o, den, floor_, head, (const float*)gate, g_ld, g_off,
                                                                  act, gate_first, w, eps, inner, group, units);
    else
        group_norm_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, o, den, floor_, head, (const bf16_t*)gate, g_ld,
                                                                   g_off, act, gate_first, w, eps, inner, group, units);
    IA_LAUNCH_CHECK("group_norm_gate");
    return 0;
}
