// Compile-time launch shapes of the streaming kernels.
#pragma once

namespace moda {

// forward and dQ kernels: waves per workgroup (32 query rows each), LDS ring stages of
// one 64-column K tile + V tile, and how many tiles ahead the global->LDS loads run.
constexpr int kRowWaves = 8;
constexpr int kRowStages = 3;
constexpr int kRowDist = 2;
constexpr int kRowBM = 32 * kRowWaves;  // query rows per workgroup

}  // namespace moda
