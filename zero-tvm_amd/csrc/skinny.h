// What the two weight-streaming kernels for 2 <= M rows share: their parameter block and tile constants.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "internal.h"

namespace ztvm {

constexpr int KS = 64;             // k per step
constexpr int WAVES = 4;           // waves per workgroup = 128 output columns

struct StreamParams {
  void* out;
  const _Float16* inp;   // activations, chunks of 8 in slot order
  const _Float16* scales;
  const uint32_t* weights;
  const _Float16* biases;
  const _Float16* xs16;  // [M][xs_stride]: hi halves, lo halves of the group sums, zero padding
  uint32_t M, N, K, row_words, spr;
  uint32_t nsteps, bias_steps, xs_stride, mtiles, ngroups, out_f32, xcd_swizzle;
  uint32_t ksplit, steps_per_split;  // k steps are dealt to ksplit workgroups, steps_per_split each
  float* partial;                    // [ksplit][M][N] when ksplit > 1
};

// The transfer-engine form of the kernel (4-bit weights, K a multiple of 128): can it run these arguments, and its
// launch. It fills p.mtiles, p.ngroups, p.ksplit and p.steps_per_split itself; partial results go to p.partial.
bool skinny_dma_supports(const MatmulArgs& a, const Tune& t);
uint32_t skinny_dma_ksplit(const MatmulArgs& a, const Tune& t);
hipError_t launch_skinny_dma(StreamParams& p, const MatmulArgs& a, const Tune& t, hipStream_t s);
// Workgroups that share the k range of one tile in the register-path kernel (skinny.hip): a function of N and K.
uint32_t skinny_reg_ksplit(const MatmulArgs& a, const Tune& t);

}  // namespace ztvm
