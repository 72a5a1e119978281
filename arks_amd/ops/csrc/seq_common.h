// Shared helpers of the sequence-state kernels (seq_*.hip).
//
// Activations are either bf16 (serving) or float (true 32-bit runs); every
// kernel is a template over that storage type and does its arithmetic in
// fp32. Small per-channel tensors (norm weights, biases, conv taps, decay
// tables) are always float.
//
// Batch layout: rows of several sequences are packed; cu_seqlens[s] is the
// first row of sequence s, seq_lens[s] its length including this step's
// rows, state_slots[s] its row in the slot-addressed state tensors (-1:
// padding — read zeros, write nothing), token_seq[t] the sequence of row t.
// A sequence whose first new position is 0 starts from zero state.
#pragma once

#include "common.h"

namespace arks {

template <typename T>
struct Act;
template <>
struct Act<float> {
  static __device__ __forceinline__ float ld(const float* p) { return *p; }
  static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
};
template <>
struct Act<bf16> {
  static __device__ __forceinline__ float ld(const bf16* p) {
    return bf16_bits_to_float(*p);
  }
  static __device__ __forceinline__ void st(bf16* p, float v) {
    *p = float_to_bf16_bits(v);
  }
};

__device__ __forceinline__ float sigmoid_f(float x) {
  return 1.f / (1.f + expf(-x));
}
__device__ __forceinline__ float silu_f(float x) { return x * sigmoid_f(x); }
__device__ __forceinline__ float softplus_f(float x) {
  return x > 20.f ? x : log1pf(expf(x));
}

struct SeqRow {
  int seq, first_row, rows, start, slot;
};

// Where row t sits in its sequence.
__device__ __forceinline__ SeqRow seq_row(int t, const int* token_seq,
                                          const int* cu, const int* seq_lens,
                                          const int* slots) {
  SeqRow r;
  r.seq = token_seq[t];
  r.first_row = cu[r.seq];
  r.rows = cu[r.seq + 1] - r.first_row;
  r.start = seq_lens[r.seq] - r.rows;
  r.slot = slots ? slots[r.seq] : -1;
  return r;
}

}  // namespace arks

// dispatch on the activation type
#define SEQ_DISPATCH_ACT(act_f32, ...)      \
  do {                                      \
    if (act_f32) {                          \
      using AT = float;                     \
      __VA_ARGS__;                          \
    } else {                                \
      using AT = arks::bf16;                \
      __VA_ARGS__;                          \
    }                                       \
  } while (0)
