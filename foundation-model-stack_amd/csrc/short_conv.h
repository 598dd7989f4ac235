// What the short causal convolutions over time share: finding a token's predecessors inside a step, and moving a
// sequence's last inputs into its state.  A convolution of `taps` taps reads the taps - 1 inputs before a token; those
// that came before the step are kept per sequence in state [slot][taps - 1][C] (the newest last, zeros before the
// sequence's start).
#pragma once

#include "common.h"

#define CONV_MAX_TAPS 8

// How many tokens of its sequence come before token t in the step, up to taps - 1 (all that a convolution of `taps`
// taps needs to know).  The candidates are loaded together, not one after another.
__device__ __forceinline__ int tokens_before(const int* __restrict__ seq_of_token, int t, int seq, int taps) {
  int prev[CONV_MAX_TAPS - 1];
#pragma unroll
  for (int d = 1; d < CONV_MAX_TAPS; ++d) prev[d - 1] = (d < taps && t - d >= 0) ? seq_of_token[t - d] : -2;
  int have = 0;
#pragma unroll
  for (int d = 1; d < CONV_MAX_TAPS; ++d)
    if (have == d - 1 && prev[d - 1] == seq) have = d;
  return have;
}

// Runs after the kernel that convolves the same step (which reads the old state).  The block of a sequence's last
// token of the step writes; new entry s is either a row of the step or an old entry above s.  x: float32 rows ld
// apart, already offset to the first convolved channel.
static __global__ void __launch_bounds__(1024)
    conv_state_kernel(const float* __restrict__ x, long ld, int taps, float* __restrict__ conv_state,
                      const int* __restrict__ seq_of_token, const int* __restrict__ slot_ids, int n_tokens, int C) {
  const int t = blockIdx.x;
  const int seq = seq_of_token[t];
  if (seq < 0) return;
  if (t + 1 < n_tokens && seq_of_token[t + 1] == seq) return;  // not the sequence's last token of the step
  const int have = tokens_before(seq_of_token, t, seq, taps);
  float* state = conv_state + (size_t)slot_ids[seq] * (taps - 1) * C;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float fresh[CONV_MAX_TAPS - 1];  // all of a channel's new entries are read before any is written
#pragma unroll
    for (int s = 0; s < CONV_MAX_TAPS - 1; ++s) {
      const int d = taps - 2 - s;  // new entry s is the input d tokens before the last one
      fresh[s] = 0.f;
      if (s < taps - 1) fresh[s] = d <= have ? x[(size_t)(t - d) * ld + c] : state[(size_t)(taps - 1 + have - d) * C + c];
    }
#pragma unroll
    for (int s = 0; s < CONV_MAX_TAPS - 1; ++s)
      if (s < taps - 1) state[(size_t)s * C + c] = fresh[s];
  }
}
