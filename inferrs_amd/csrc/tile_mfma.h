// The tile of tile_fma.h on the matrix cores, for bfloat16 operands: out[i][j] = sum_k x_i[k] * w[j][k] for 32
// gathered rows x 64 output features a block of four waves.  k comes through shared memory in chunks of 64 (rows of
// 144 bytes: the 16-byte operand reads of 16 lanes then meet every bank once), the next chunk is on its way from
// memory into registers while this one is multiplied.  A wave owns 16 features and both tiles of 16 rows.
//
// v_mfma_f32_16x16x32_bf16: lane l supplies row (l % 16) of A and column (l % 16) of B with the eight k values
// (l / 16) * 8 .. + 8 and receives D[4 (l / 16) + i][l % 16].  A = the weights' rows, B = the gathered rows, so a lane
// ends with four neighbouring features of one row.  Every output is a sum over k in the same order whatever rows
// share the tile.  k a multiple of 8, rows and weights 16-byte aligned (the launchers check).
#pragma once

#include "common.h"

typedef __bf16 tm_bf16x8 __attribute__((ext_vector_type(8)));
typedef float tm_f32x4 __attribute__((ext_vector_type(4)));

#define IA_MM 32
#define IA_MN 64
#define IA_MK 64
#define IA_MROW 72          // elements of a staged row (64 and 8 of padding)

struct TileSharedMfma {
    __attribute__((aligned(16))) uint16_t xs[IA_MM][IA_MROW];
    __attribute__((aligned(16))) uint16_t ws[IA_MN][IA_MROW];
    __attribute__((aligned(16))) uint16_t ws2[IA_MN][IA_MROW];
};

// acc[rt]: features 16 (wave) + 4 (lane / 16) + i of row 16 rt + lane % 16.
template <bool DUAL, typename RowFn>
__device__ __forceinline__ void tile_product_mfma(tm_f32x4 (&acc)[2], tm_f32x4 (&acc2)[2], TileSharedMfma& sh, RowFn xrow,
                                                  const bf16_t* __restrict__ w, const bf16_t* __restrict__ w2, int n_valid,
                                                  int K, long long ldw) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
        acc[rt] = (tm_f32x4){0.f, 0.f, 0.f, 0.f};
        acc2[rt] = (tm_f32x4){0.f, 0.f, 0.f, 0.f};
    }
    const int xi = tid >> 3, piece = tid & 7;              // the row and 16-byte piece this thread stages
    const bf16_t* xp = xrow(xi);
    const bf16_t* wp[2];
    const bf16_t* wp2[2];
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const int j = xi + 32 * r;
        wp[r] = j < n_valid ? w + (long long)j * ldw : nullptr;
        wp2[r] = (DUAL && j < n_valid) ? w2 + (long long)j * ldw : nullptr;
    }
    uint4 rx, rw[2], rw2[2];
    auto fetch = [&](int k0) {
        const int k = k0 + piece * 8;
        const bool in = k < K;
        rx = (xp != nullptr && in) ? *reinterpret_cast<const uint4*>(xp + k) : zero;
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            rw[r] = (wp[r] != nullptr && in) ? *reinterpret_cast<const uint4*>(wp[r] + k) : zero;
            if (DUAL) rw2[r] = (wp2[r] != nullptr && in) ? *reinterpret_cast<const uint4*>(wp2[r] + k) : zero;
        }
    };
    fetch(0);
    for (int k0 = 0; k0 < K; k0 += IA_MK) {
        __syncthreads();
        *reinterpret_cast<uint4*>(&sh.xs[xi][piece * 8]) = rx;
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            *reinterpret_cast<uint4*>(&sh.ws[xi + 32 * r][piece * 8]) = rw[r];
            if (DUAL) *reinterpret_cast<uint4*>(&sh.ws2[xi + 32 * r][piece * 8]) = rw2[r];
        }
        __syncthreads();
        if (k0 + IA_MK < K) fetch(k0 + IA_MK);
#pragma unroll
        for (int ks = 0; ks < IA_MK / 32; ++ks) {
            const int ko = ks * 32 + (lane >> 4) * 8;
            const tm_bf16x8 a = *reinterpret_cast<const tm_bf16x8*>(&sh.ws[16 * wave + (lane & 15)][ko]);
            tm_bf16x8 a2;
            if (DUAL) a2 = *reinterpret_cast<const tm_bf16x8*>(&sh.ws2[16 * wave + (lane & 15)][ko]);
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
                const tm_bf16x8 b = *reinterpret_cast<const tm_bf16x8*>(&sh.xs[16 * rt + (lane & 15)][ko]);
                acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[rt], 0, 0, 0);
                if (DUAL) acc2[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2, b, acc2[rt], 0, 0, 0);
            }
        }
    }
}

static inline bool tile_mfma_aligned(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
