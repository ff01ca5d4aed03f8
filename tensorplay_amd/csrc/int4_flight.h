// Host interface of the all-in-flight matrix-core int4 kernel (int4_mfma_flight_kernel.h, built in int4_flight.hip).
#pragma once

#include "tpq_common.h"

namespace tpq {

struct FlightWeights {
    const void* packed[4];  // device layout, innerKTiles = 2
    const void* sz[4];      // [K/group][N] (scale, zero) pairs of the activation dtype
    void* y[4];             // [rows][N]
    int N[4];
    int count;              // 1..4 weights; pair: 2 weights of the same N, one output y[0]
    const void* norm_weight;  // not null: the activations are RMS-normalized first, weights [K] of the activation dtype
    float norm_eps;
};

// 2..16 activation rows, 16-bit activations.  Returns false when the shape is not one of the built cases (nothing
// launched, *rc untouched); true after a launch attempt, *rc = TPQ_OK or the error.
// pair: out = silu_mul(x . W[0]^T, x . W[1]^T); residual (one weight, not a pair; may be null): added to the rounded output.
bool flight_launch(int dtype, const void* x, int rows, const FlightWeights& weights, int K, int group, bool pair,
                   const void* residual, hipStream_t stream, int* rc);

// The int8 weight-only product (w: [N][K] int8, scales: [N] float, y = (x . w^T) * scale) on the same structure
// (int8pack_flight_kernel.h): 3..16 rows of 16-bit activations.  Returns false when the shape is not built.
bool flight_launch_int8pack(int dtype, const void* x, int rows, const int8_t* w, const float* scales, void* y, int N, int K,
                            hipStream_t stream, int* rc);

}  // namespace tpq
