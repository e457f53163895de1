// The tile of tile_fma.h on the matrix cores, for bfloat16 operands: out[i][j] = sum_k x_i[k] * w[j][k] for
// 16 RT gathered rows x 64 FT output features a block of four waves.  k comes through shared memory in chunks of KC
// (rows padded by 16 bytes: the 16-byte operand reads of 16 lanes then meet every bank once), the next chunk is on its
// way from memory into registers while this one is multiplied.  A wave owns 16 FT features and all RT tiles of 16 rows.
// Shapes in use: 32 rows x 64 features (few rows a group) and 64 rows x 128 features (many rows a group: every
// operand read serves more products), k in chunks of 64.  The routed experts store their weights as tiles of 64
// features x 64 k values (`product_tiled`): a wave's load is then 1 KB in one piece, where rows of the plain layout
// make it eight pieces of 128 bytes from eight rows, which the compute unit's address unit takes far longer over.
//
// v_mfma_f32_16x16x32_bf16: lane l supplies row (l % 16) of A and column (l % 16) of B with the eight k values
// (l / 16) * 8 .. + 8 and receives D[4 (l / 16) + i][l % 16].  A = the weights' rows, B = the gathered rows, so a lane
// ends with four neighbouring features of one row.  Every output is a sum over k in the same order whatever rows
// share the tile and whichever shape runs.  k a multiple of 8, rows and weights 16-byte aligned (the launchers check).
#pragma once

#include "common.h"

typedef __bf16 tm_bf16x8 __attribute__((ext_vector_type(8)));
typedef float tm_f32x4 __attribute__((ext_vector_type(4)));
// 16 bytes on their way from memory to shared memory: the compiler's own vector type, which stays in registers (the
// runtime's uint4 is a class, and arrays of it have ended up in scratch or shared memory)
typedef uint32_t tm_u32x4 __attribute__((ext_vector_type(4)));

template <int RT, int FT, int KC, bool DUAL>
struct TileMfma {
    static constexpr int ROWS = 16 * RT, FEATURES = 64 * FT, ROW = KC + 8, PPR = KC / 8;
    static constexpr int NX = ROWS * PPR / 256, NW = FEATURES * PPR / 256;
    static_assert(ROWS * PPR % 256 == 0 && FEATURES * PPR % 256 == 0, "a block of 256 threads stages whole rounds");

    struct Shared {
        __attribute__((aligned(16))) uint16_t xs[ROWS][ROW];
        __attribute__((aligned(16))) uint16_t ws[FEATURES][ROW];
        __attribute__((aligned(16))) uint16_t ws2[DUAL ? FEATURES : 1][ROW];
    };

    // acc[ft][rt]: features 16 (FT wave + ft) + 4 (lane / 16) + i of row 16 rt + lane % 16.
    template <typename RowFn>
    static __device__ __forceinline__ void product(tm_f32x4 (&acc)[FT][RT], tm_f32x4 (&acc2)[FT][RT], Shared& sh, RowFn xrow,
                                                   const bf16_t* __restrict__ w, const bf16_t* __restrict__ w2, int n_valid,
                                                   int K, long long ldw) {
        const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
        const tm_u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int ft = 0; ft < FT; ++ft)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                acc[ft][rt] = (tm_f32x4){0.f, 0.f, 0.f, 0.f};
                acc2[ft][rt] = (tm_f32x4){0.f, 0.f, 0.f, 0.f};
            }
        const int piece = tid % PPR, row0 = tid / PPR;      // this thread stages rows row0 + i * (256 / PPR)
        const bf16_t* xp[NX];
        const bf16_t* wp[NW];
        const bf16_t* wp2[NW];
#pragma unroll
        for (int i = 0; i < NX; ++i) xp[i] = xrow(row0 + i * (256 / PPR));
#pragma unroll
        for (int i = 0; i < NW; ++i) {
            const int j = row0 + i * (256 / PPR);
            wp[i] = j < n_valid ? w + (long long)j * ldw : nullptr;
            wp2[i] = (DUAL && j < n_valid) ? w2 + (long long)j * ldw : nullptr;
        }
        tm_u32x4 rx[NX], rw[NW], rw2[NW];
        auto fetch = [&](int k0) {
            const int k = k0 + piece * 8;
            const bool in = k < K;
#pragma unroll
            for (int i = 0; i < NX; ++i) rx[i] = (xp[i] != nullptr && in) ? *reinterpret_cast<const tm_u32x4*>(xp[i] + k) : zero;
#pragma unroll
            for (int i = 0; i < NW; ++i) {
                rw[i] = (wp[i] != nullptr && in) ? *reinterpret_cast<const tm_u32x4*>(wp[i] + k) : zero;
                if (DUAL) rw2[i] = (wp2[i] != nullptr && in) ? *reinterpret_cast<const tm_u32x4*>(wp2[i] + k) : zero;
            }
        };
        fetch(0);
        for (int k0 = 0; k0 < K; k0 += KC) {
            __syncthreads();
#pragma unroll
            for (int i = 0; i < NX; ++i) *reinterpret_cast<tm_u32x4*>(&sh.xs[row0 + i * (256 / PPR)][piece * 8]) = rx[i];
#pragma unroll
            for (int i = 0; i < NW; ++i) {
                *reinterpret_cast<tm_u32x4*>(&sh.ws[row0 + i * (256 / PPR)][piece * 8]) = rw[i];
                if (DUAL) *reinterpret_cast<tm_u32x4*>(&sh.ws2[row0 + i * (256 / PPR)][piece * 8]) = rw2[i];
            }
            __syncthreads();
            if (k0 + KC < K) fetch(k0 + KC);
#pragma unroll
            for (int ks = 0; ks < KC / 32; ++ks) {
                const int ko = ks * 32 + (lane >> 4) * 8;
                tm_bf16x8 b[RT];
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) b[rt] = *reinterpret_cast<const tm_bf16x8*>(&sh.xs[16 * rt + (lane & 15)][ko]);
#pragma unroll
                for (int ft = 0; ft < FT; ++ft) {
                    const int fr = 16 * (wave * FT + ft) + (lane & 15);
                    const tm_bf16x8 a = *reinterpret_cast<const tm_bf16x8*>(&sh.ws[fr][ko]);
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) acc[ft][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[rt], acc[ft][rt], 0, 0, 0);
                    if (DUAL) {
                        const tm_bf16x8 a2 = *reinterpret_cast<const tm_bf16x8*>(&sh.ws2[fr][ko]);
#pragma unroll
                        for (int rt = 0; rt < RT; ++rt)
                            acc2[ft][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2, b[rt], acc2[ft][rt], 0, 0, 0);
                    }
                }
            }
        }
    }

    // Chunk c of the thread's pieces of the rows and of the tiled weights, into registers.  No load is conditional:
    // a row that does not exist reads the tile's first row, a feature block that does not exist the last one that does
    // (their outputs are dropped), and a piece beyond K reads the row's last piece (the weights' padding there is zero).
    static __device__ __forceinline__ void fetch_tiled(tm_u32x4 (&rx)[NX], tm_u32x4 (&rw)[NW], tm_u32x4 (&rw2)[NW],
                                                       const bf16_t* const (&xp)[NX], const bf16_t* wbase,
                                                       const bf16_t* wbase2, long long fb_stride, int fb_left, int piece,
                                                       int c, int K) {
        const int k = min(c * KC + piece * 8, K - 8);
#pragma unroll
        for (int i = 0; i < NX; ++i) rx[i] = *reinterpret_cast<const tm_u32x4*>(xp[i] + k);
#pragma unroll
        for (int i = 0; i < NW; ++i) {
            const long long at = min(i / 2, fb_left - 1) * fb_stride + (i % 2) * 2048 + (long long)c * 4096;
            rw[i] = *reinterpret_cast<const tm_u32x4*>(wbase + at);
            if (DUAL) rw2[i] = *reinterpret_cast<const tm_u32x4*>(wbase2 + at);
        }
    }

    // The same product with the weights stored as tiles: 64 features x 64 k values contiguous (8 KB), a matrix as
    // [feature blocks][k chunks][64][64], zero-padded in both directions, so that every load of a wave is 1 KB in one
    // piece and needs no bounds.  `wt` points at the block's first feature block (k chunk 0), `wt2` likewise in the
    // second matrix; `fb_left`: feature blocks that exist from there on; `chunks`: k chunks.  KC is 64.
    template <typename RowFn>
    static __device__ __forceinline__ void product_tiled(tm_f32x4 (&acc)[FT][RT], tm_f32x4 (&acc2)[FT][RT], Shared& sh,
                                                         RowFn xrow, const bf16_t* __restrict__ wt,
                                                         const bf16_t* __restrict__ wt2, int fb_left, int chunks, int K) {
        static_assert(KC == 64, "tiles of the stored weights hold 64 k values");
        const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
        const tm_u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int ft = 0; ft < FT; ++ft)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                acc[ft][rt] = (tm_f32x4){0.f, 0.f, 0.f, 0.f};
                acc2[ft][rt] = (tm_f32x4){0.f, 0.f, 0.f, 0.f};
            }
        const int piece = tid % PPR, row0 = tid / PPR;
        const bf16_t* xp[NX];
#pragma unroll
        for (int i = 0; i < NX; ++i) {
            xp[i] = xrow(row0 + i * (256 / PPR));
            if (xp[i] == nullptr) xp[i] = xrow(0);          // (a tile has a first row)
        }
        // rows row0 + 32 i of the block's 64 FT weight rows: feature block i / 2, and inside it the thread's own 16 bytes
        const long long fb_stride = (long long)chunks * 4096;
        const bf16_t* wbase = wt + tid * 8;
        const bf16_t* wbase2 = wt2 + tid * 8;
        tm_u32x4 rx[NX], rw[NW], rw2[NW];
        fetch_tiled(rx, rw, rw2, xp, wbase, wbase2, fb_stride, fb_left, piece, 0, K);
        for (int c = 0; c < chunks; ++c) {
            __syncthreads();
#pragma unroll
            for (int i = 0; i < NX; ++i) *reinterpret_cast<tm_u32x4*>(&sh.xs[row0 + i * (256 / PPR)][piece * 8]) = rx[i];
#pragma unroll
            for (int i = 0; i < NW; ++i) {
                *reinterpret_cast<tm_u32x4*>(&sh.ws[row0 + i * (256 / PPR)][piece * 8]) = rw[i];
                if (DUAL) *reinterpret_cast<tm_u32x4*>(&sh.ws2[row0 + i * (256 / PPR)][piece * 8]) = rw2[i];
            }
            __syncthreads();
            if (c + 1 < chunks) fetch_tiled(rx, rw, rw2, xp, wbase, wbase2, fb_stride, fb_left, piece, c + 1, K);
#pragma unroll
            for (int ks = 0; ks < KC / 32; ++ks) {
                const int ko = ks * 32 + (lane >> 4) * 8;
                tm_bf16x8 b[RT];
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) b[rt] = *reinterpret_cast<const tm_bf16x8*>(&sh.xs[16 * rt + (lane & 15)][ko]);
#pragma unroll
                for (int ft = 0; ft < FT; ++ft) {
                    const int fr = 16 * (wave * FT + ft) + (lane & 15);
                    const tm_bf16x8 a = *reinterpret_cast<const tm_bf16x8*>(&sh.ws[fr][ko]);
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) acc[ft][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[rt], acc[ft][rt], 0, 0, 0);
                    if (DUAL) {
                        const tm_bf16x8 a2 = *reinterpret_cast<const tm_bf16x8*>(&sh.ws2[fr][ko]);
#pragma unroll
                        for (int rt = 0; rt < RT; ++rt)
                            acc2[ft][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2, b[rt], acc2[ft][rt], 0, 0, 0);
                    }
                }
            }
        }
    }

    // calls f(row of the tile, feature of the tile, ft, rt, i) for every output this lane holds
    template <typename F>
    static __device__ __forceinline__ void each(F f) {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int ft = 0; ft < FT; ++ft)
#pragma unroll
                for (int i = 0; i < 4; ++i) f(16 * rt + (lane & 15), 16 * (wave * FT + ft) + 4 * (lane >> 4) + i, ft, rt, i);
    }
};

static inline bool tile_mfma_aligned(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
