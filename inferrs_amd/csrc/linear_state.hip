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

extern "C" int ia_exp_gates(float* log_a, float* b, float* floor_, float* state, long long row_floats, long long m_off,
                            const void* proj, long long p_ld, int i_off, int f_off, const float* bias_i,
                            const float* bias_f, float cap, const int* cu_tokens, const int* state_slots, int H,
                            int n_seqs, int dtype, hipStream_t stream) {
    IA_CHECK(H > 0 && n_seqs >= 0 && cap > 0.f && i_off >= 0 && f_off >= 0 && i_off + H <= p_ld && f_off + H <= p_ld,
             "exp_gates: bad sizes heads=%d cap=%g", H, (double)cap);
    IA_CHECK(m_off >= 0 && m_off + H <= row_floats, "exp_gates: the maxima do not fit the state row");
    if (n_seqs == 0) return 0;
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

// ---- the recurrence, token by token -----------------------------------------------------------------------------------
// A block owns a (request, head, tile of S's columns) and walks the request's tokens in order.  A column j of S is
// shared by P neighbouring lanes, each with LS_R of the column's `dim` entries in registers; the lanes add up q . S[:, j]
// by a butterfly.  The next token's operands are asked for while this one is computed.  Nothing in the order of the sums
// depends on how the tokens were cut into steps or on the batch.
#define LS_R 8
#define LS_THREADS 256

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
};

template <typename T>
__global__ __launch_bounds__(LS_THREADS) void linear_scan_kernel(const ScanArgs a) {
    const int P = a.P;
    const int p = threadIdx.x % P, jj = threadIdx.x / P;
    const int h = blockIdx.y, seq = blockIdx.z;
    const int vt = a.vdim + (a.den != nullptr ? 1 : 0);           // columns of S
    const int j = blockIdx.x * a.cols + jj;
    const bool live = j < vt;
    const bool ones = j >= a.vdim;                                // the column whose value is always 1
    const int first = a.cu_tokens[seq], last = a.cu_tokens[seq + 1];
    const int qh = h / (a.H / a.q_heads), kh = h / (a.H / a.k_heads);
    const int i0 = p * LS_R;
    const T* q = (const T*)a.q + a.q_off + (long long)qh * a.dim + i0;
    const T* k = (const T*)a.k + a.k_off + (long long)kh * a.dim + i0;
    const T* v = (const T*)a.v + a.v_off + (long long)h * a.vdim + (ones || !live ? 0 : j);
    float* srow = a.state + (long long)a.state_slots[seq] * a.row_floats + a.s_off +
                  ((long long)h * vt + (live ? j : 0)) * a.dim + i0;
    float S[LS_R];
#pragma unroll
    for (int r = 0; r < LS_R; ++r) S[r] = (live && i0 + r < a.dim) ? srow[r] : 0.f;
    const float skip = a.skip != nullptr ? a.skip[h] : 0.f;

    float qn[LS_R], kn[LS_R], vn = 0.f, an = 0.f, bn = 1.f;
    auto fetch = [&](int t) {
#pragma unroll
        for (int r = 0; r < LS_R; ++r) {
            const bool in = i0 + r < a.dim;
            qn[r] = in ? ld(q + (long long)t * a.q_ld + r) : 0.f;
            kn[r] = in ? ld(k + (long long)t * a.k_ld + r) : 0.f;
        }
        vn = ones ? 1.f : ld(v + (long long)t * a.v_ld);
        an = a.log_a[a.a_per_token ? (long long)t * a.H + h : h];
        bn = a.b != nullptr ? a.b[(long long)t * a.H + h] : 1.f;
    };
    if (first < last) fetch(first);
    for (int t = first; t < last; ++t) {
        float qc[LS_R], kc[LS_R];
#pragma unroll
        for (int r = 0; r < LS_R; ++r) { qc[r] = qn[r] * a.q_scale; kc[r] = kn[r] * a.k_scale; }
        const float vc = vn, decay = a.a_per_token ? expf(an) : an, bv = bn * vn;
        if (t + 1 < last) fetch(t + 1);
        float part = 0.f;
#pragma unroll
        for (int r = 0; r < LS_R; ++r) {
            S[r] = fmaf(decay, S[r], bv * kc[r]);
            part = fmaf(S[r], qc[r], part);
        }
        for (int o = P / 2; o > 0; o >>= 1) part += __shfl_xor(part, o, IA_WAVE);
        if (p == 0 && live) {
            if (ones) a.den[(long long)t * a.H + h] = part;
            else a.out[((long long)t * a.H + h) * a.vdim + j] = fmaf(skip, vc, part);
        }
    }
    if (live)
#pragma unroll
        for (int r = 0; r < LS_R; ++r)
            if (i0 + r < a.dim) srow[r] = S[r];
}

extern "C" int ia_linear_scan(float* out, float* den, float* state, long long row_floats, long long s_off,
                              const void* q, long long q_ld, int q_off, int q_heads,
                              const void* k, long long k_ld, int k_off, int k_heads,
                              const void* v, long long v_ld, int v_off,
                              const float* log_a, int a_per_token, const float* b, const float* skip,
                              const int* cu_tokens, const int* state_slots, int n_seqs, int H, int dim, int vdim,
                              float q_scale, float k_scale, int dtype, hipStream_t stream) {
    IA_CHECK(n_seqs >= 0 && H > 0 && dim > 0 && vdim > 0, "linear_scan: bad sizes heads=%d dim=%d vdim=%d", H, dim, vdim);
    IA_CHECK(dim <= LS_R * IA_WAVE, "linear_scan: a key size of %d is beyond %d", dim, LS_R * IA_WAVE);
    IA_CHECK(q_heads > 0 && k_heads > 0 && H % q_heads == 0 && H % k_heads == 0,
             "linear_scan: %d heads over %d query and %d key heads", H, q_heads, k_heads);
    const int vt = vdim + (den != nullptr ? 1 : 0);
    IA_CHECK(s_off >= 0 && s_off + (long long)H * vt * dim <= row_floats, "linear_scan: the matrices do not fit the state row");
    IA_CHECK(q_off >= 0 && q_off + (long long)q_heads * dim <= q_ld && k_off >= 0 && k_off + (long long)k_heads * dim <= k_ld &&
             v_off >= 0 && v_off + (long long)H * vdim <= v_ld, "linear_scan: q, k or v lie outside their rows");
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
    const dim3 grid((unsigned)((vt + a.cols - 1) / a.cols), (unsigned)H, (unsigned)n_seqs);
    if (dtype == IA_F32) linear_scan_kernel<float><<<grid, LS_THREADS, 0, stream>>>(a);
    else linear_scan_kernel<bf16_t><<<grid, LS_THREADS, 0, stream>>>(a);
    IA_LAUNCH_CHECK("linear_scan");
    return 0;
}

// ---- what follows the recurrence: a norm a group of features, a gate, an optional division --------------------------
//     y = o / (max(|den|, floor) + 1e-6)        (with den: the matrix memory's normaliser, a (token, head))
//     y = y * act(g)                            (gate_first: the gate comes before the norm)
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
