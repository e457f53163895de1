// A tile of a matrix product on the vector units, for products whose rows are gathered or whose weights change
// from group to group (heads, blocks of a block-diagonal matrix, routed experts): out[i][j] = sum_k x_i[k] * w[j][k].
// A block of 256 threads owns 32 rows x 64 output features; k comes through shared memory in chunks of 16.  Every
// output is ONE chain of fused multiply-adds with k ascending, whatever else is in the tile: a row's result does not
// depend on which rows stand beside it.  Operands of any storage type, sums in 32-bit.
#pragma once

#include "common.h"

#define IA_TM 32
#define IA_TN 64
#define IA_TK 16

struct TileShared {
    float xs[IA_TK][IA_TM + 1];
    float ws[IA_TK][IA_TN + 1];
    float ws2[IA_TK][IA_TN + 1];
};

// `xrow(i)`: pointer to row i of the tile (i in 0..31) or nullptr for a row that does not exist; `w` points at the
// first of the tile's 64 weight rows ([.., ldw] each), of which `n_valid` exist; with DUAL a second matrix `w2` of the
// same shape is multiplied with the same rows into `acc2`.  Thread t owns rows 2 (t / 16) + {0, 1} and features
// 4 (t % 16) + {0..3}.
template <typename TX, typename TW, bool DUAL, typename RowFn>
__device__ __forceinline__ void tile_product(float (&acc)[2][4], float (&acc2)[2][4], TileShared& sh, RowFn xrow,
                                             const TW* __restrict__ w, const TW* __restrict__ w2, int n_valid, int K,
                                             long long ldw) {
    const int tid = threadIdx.x;
    const int ty = tid >> 4, tx = tid & 15;
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[a][b] = acc2[a][b] = 0.f;
    // what this thread stages: two elements of x (row xi, k xk and xk + 8), four of w (row wj + 16 r, k wk)
    const int xi = tid >> 3, xk = tid & 7;
    const TX* xp = xrow(xi);
    const int wk = tid & 15, wj = tid >> 4;
    for (int k0 = 0; k0 < K; k0 += IA_TK) {
        __syncthreads();
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int k = k0 + xk + 8 * r;
            sh.xs[xk + 8 * r][xi] = (xp != nullptr && k < K) ? ld(xp + k) : 0.f;
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int j = wj + 16 * r, k = k0 + wk;
            const bool ok = j < n_valid && k < K;
            sh.ws[wk][j] = ok ? ld(w + (long long)j * ldw + k) : 0.f;
            if (DUAL) sh.ws2[wk][j] = ok ? ld(w2 + (long long)j * ldw + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < IA_TK; ++kk) {
            const float a0 = sh.xs[kk][2 * ty], a1 = sh.xs[kk][2 * ty + 1];
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const float wv = sh.ws[kk][4 * tx + b];
                acc[0][b] = fmaf(a0, wv, acc[0][b]);
                acc[1][b] = fmaf(a1, wv, acc[1][b]);
                if (DUAL) {
                    const float wv2 = sh.ws2[kk][4 * tx + b];
                    acc2[0][b] = fmaf(a0, wv2, acc2[0][b]);
                    acc2[1][b] = fmaf(a1, wv2, acc2[1][b]);
                }
            }
        }
    }
}
