// A tile product on the matrix cores for matrices picked per expert or per head (bfloat16):
// a workgroup of four wavefronts computes 64 rows x 64 CT columns of a w^T, a wavefront 16 CT of the
// columns for all the rows, operands straight from memory, sums in 32-bit, k in steps
// of 32 in a fixed order.  The weights are the first operand, so that a lane ends up with four
// neighbouring columns of one row.  K a multiple of 32; rows of a and w 16-byte aligned.
#pragma once
#include "common.h"

typedef __bf16 mr_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 mr_bf16x4 __attribute__((ext_vector_type(4)));
typedef float mr_f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int mr_u32x4 __attribute__((ext_vector_type(4)));

#define MR_ROWS 64
#define MR_COLS 64

// sums[s][ct][rt][r]: stream s, column tile ct of the wavefront, row rt * 16 + (lane & 15), column
// (first column of the tile) + 4 (lane >> 4) + r.  a_row[rt]: this lane's row of a for row tile rt (null:
// none); w_row[s][ct]: this lane's weight row (column of the tile + (lane & 15)) of stream s (null: none).
// A wavefront with CT column tiles uses every operand of a it has loaded CT times.
// K is walked in pieces of 64: a lane asks for 32 bytes in a run of each of its rows (its operands of
// the piece's two matrix instructions), all of a piece's loads issued while the piece before is
// multiplied.  The values of k are thereby dealt to the instructions in another order than they lie in
// (lane quad qd, instruction i of a piece: k0 + 16 qd + 8 i ..+8), the same order for both operands
// and for every row, whatever else is in the batch.
template <int STREAMS, int CT>
__device__ __forceinline__ void mfma_rows_product(const __bf16* const (&a_row)[4], int row_tiles,
                                                  const __bf16* const (&w_row)[STREAMS][CT], int K,
                                                  mr_f32x4 (&sums)[STREAMS][CT][4]) {
    constexpr int NI = 2;      // matrix instructions a piece: 64 values of k, 32 bytes a lane and row
    const int qd = (threadIdx.x & 63) >> 4;
#pragma unroll
    for (int s = 0; s < STREAMS; ++s)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) sums[s][ct][rt] = mr_f32x4{0.f, 0.f, 0.f, 0.f};
    const mr_u32x4 zero = {0u, 0u, 0u, 0u};
    auto load = [&](int k0, mr_u32x4 (&wf)[STREAMS][CT][NI], mr_u32x4 (&af)[4][NI]) __attribute__((always_inline)) {
        const int k = k0 + qd * (8 * NI);
#pragma unroll
        for (int s = 0; s < STREAMS; ++s)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                for (int i = 0; i < NI; ++i)
                    wf[s][ct][i] = w_row[s][ct] && k + 8 * i < K ? *reinterpret_cast<const mr_u32x4*>(w_row[s][ct] + k + 8 * i) : zero;
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int i = 0; i < NI; ++i)
                af[rt][i] = rt < row_tiles && a_row[rt] && k + 8 * i < K ? *reinterpret_cast<const mr_u32x4*>(a_row[rt] + k + 8 * i) : zero;
    };
    auto multiply = [&](const mr_u32x4 (&wf)[STREAMS][CT][NI], const mr_u32x4 (&af)[4][NI]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int s = 0; s < STREAMS; ++s)
#pragma unroll
                for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                    for (int rt = 0; rt < 4; ++rt)
                        if (rt < row_tiles)
                            sums[s][ct][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(mr_bf16x8, wf[s][ct][i]),
                                                                                    __builtin_bit_cast(mr_bf16x8, af[rt][i]),
                                                                                    sums[s][ct][rt], 0, 0, 0);
    };
    // two sets of operand registers: a piece is asked for while the piece before is multiplied
    mr_u32x4 wf0[STREAMS][CT][NI], af0[4][NI], wf1[STREAMS][CT][NI], af1[4][NI];
    constexpr int PIECE = 32 * NI;
    load(0, wf0, af0);
    for (int k0 = 0; k0 < K; k0 += 2 * PIECE) {
        load(k0 + PIECE, wf1, af1);          // (beyond K: zeros, nothing read)
        multiply(wf0, af0);
        load(k0 + 2 * PIECE, wf0, af0);
        if (k0 + PIECE < K) multiply(wf1, af1);
    }
}
