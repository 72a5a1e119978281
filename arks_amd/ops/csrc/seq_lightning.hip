// Lightning (linear) attention with one scalar decay per head:
//   S_t = decay * S_{t-1} + k_t v_t^T,  o_t = S_t^T q_t,  q,k,v = silu(.)
// S is a [D x V] fp32 matrix per head and sequence, kept in a slot-addressed
// state tensor between steps.
//
// Two input conventions (template MODE): 0 — q, k and v pass through silu;
// 1 — plain rows, q and k turned by their position over their first 2*n_rot
// dims (pairs (2i, 2i+1) when interleaved, (i, i+n_rot) otherwise; angle =
// position * freq[i], fp32) and k multiplied by k_scale after that.
//
// General kernel: one wave per (sequence, head, 64 value columns); lane c
// owns column c of S in registers and walks the sequence's rows in order.
// The row's silu(q), silu(k) are staged in LDS once per row for all lanes.
#include "seq_common.h"

namespace arks {

// Element d of a head's q or k row turned by `pos` (MODE 1 loads).
template <typename AT>
__device__ __forceinline__ float rotated_ld(const AT* row, int d, float pos,
                                            const float* freq, int n_rot,
                                            int interleaved) {
  const float x = Act<AT>::ld(row + d);
  if (d >= 2 * n_rot) return x;
  const int i = interleaved ? d >> 1 : (d < n_rot ? d : d - n_rot);
  const bool first = interleaved ? !(d & 1) : d < n_rot;
  const int dp = interleaved ? d ^ 1 : (first ? d + n_rot : d - n_rot);
  const float y = Act<AT>::ld(row + dp);
  float sn, cs;
  sincosf(pos * freq[i], &sn, &cs);
  return first ? x * cs - y * sn : x * cs + y * sn;
}

template <typename AT, int DMAX, int MODE>
__global__ __launch_bounds__(64) void lightning_scan_kernel(
    float* __restrict__ out, const AT* __restrict__ q, const AT* __restrict__ k,
    const AT* __restrict__ v, int64_t ldq, int64_t ldk, int64_t ldv,
    const float* __restrict__ decay, float* __restrict__ state,
    const int* __restrict__ cu, const int* __restrict__ seq_lens,
    const int* __restrict__ slots, int H, int D, int V,
    const int64_t* __restrict__ positions, const float* __restrict__ freq,
    int n_rot, int interleaved, float k_scale) {
  __shared__ float q_s[2][DMAX];
  __shared__ float k_s[2][DMAX];
  const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int col = blockIdx.z * 64 + lane;
  const int a = cu[s], rows = cu[s + 1] - a;
  if (rows == 0) return;
  const int start = seq_lens[s] - rows;
  const int slot = slots[s];
  const bool live = col < V;
  const float lam = decay[h];
  float S[DMAX];
  float* sp = state + (((int64_t)(slot < 0 ? 0 : slot) * H + h) * D) * V + col;
  const bool has_state = start > 0 && slot >= 0 && live;
#pragma unroll
  for (int d = 0; d < DMAX; ++d)
    S[d] = (has_state && d < D) ? sp[(int64_t)d * V] : 0.f;
  for (int r = 0; r < rows; ++r) {
    const int t = a + r;
    const int buf = r & 1;  // double buffer: one barrier per row
    if (MODE == 0) {
      for (int d = lane; d < D; d += 64) {
        q_s[buf][d] = silu_f(Act<AT>::ld(q + (int64_t)t * ldq + (int64_t)h * D + d));
        k_s[buf][d] = silu_f(Act<AT>::ld(k + (int64_t)t * ldk + (int64_t)h * D + d));
      }
    } else {
      const float pos = (float)positions[t];
      for (int d = lane; d < D; d += 64) {
        q_s[buf][d] = rotated_ld<AT>(q + (int64_t)t * ldq + (int64_t)h * D, d,
                                     pos, freq, n_rot, interleaved);
        k_s[buf][d] = k_scale * rotated_ld<AT>(k + (int64_t)t * ldk + (int64_t)h * D,
                                               d, pos, freq, n_rot, interleaved);
      }
    }
    float vv = 0.f;
    if (live) {
      vv = Act<AT>::ld(v + (int64_t)t * ldv + (int64_t)h * V + col);
      if (MODE == 0) vv = silu_f(vv);
    }
    __syncthreads();
    float o = 0.f;
#pragma unroll
    for (int d = 0; d < DMAX; ++d) {
      if (d < D) {
        S[d] = lam * S[d] + k_s[buf][d] * vv;
        o += S[d] * q_s[buf][d];
      }
    }
    if (live) out[((int64_t)t * H + h) * V + col] = o;
  }
  if (slot >= 0 && live) {
#pragma unroll
    for (int d = 0; d < DMAX; ++d)
      if (d < D) sp[(int64_t)d * V] = S[d];
  }
}

// Chunk-parallel prefill, middle step (see scan_combine_kernel in
// seq_mamba.hip): part[k] = end state of chunk k scanned from zero; replace
// it by the state at the chunk's start, carrying decay^(rows of the chunk)
// across each chunk. chunk_rows[k] = rows of chunk k.
__global__ __launch_bounds__(256) void lightning_combine_kernel(
    float* __restrict__ part, const float* __restrict__ decay,
    float* __restrict__ state, const int* __restrict__ chunk_off,
    const int* __restrict__ chunk_rows, const int* __restrict__ cu,
    const int* __restrict__ seq_lens, const int* __restrict__ slots, int H,
    int D, int V, int transposed) {
  const int DV = D * V;
  const int s = blockIdx.y;
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= (int64_t)H * DV) return;
  // the scratch states may be stored [v][d]; the slot state is [d][v]
  int64_t se = e;
  if (transposed) {
    const int hh = (int)(e / DV), rem = (int)(e - (int64_t)hh * DV);
    se = (int64_t)hh * DV + (int64_t)(rem % D) * V + rem / D;
  }
  const int rows = cu[s + 1] - cu[s];
  if (rows == 0) return;
  const int start = seq_lens[s] - rows;
  const int slot = slots[s];
  const float lam = decay[e / DV];
  float carry = (start > 0 && slot >= 0) ? state[(int64_t)slot * H * DV + se] : 0.f;
  // the next chunk's value is loaded before this chunk's slot is rewritten,
  // and decay^rows is evaluated again only when the row count changes
  // (every chunk but a sequence's last has the same)
  const int k0 = chunk_off[s], k1 = chunk_off[s + 1];
  const int64_t stride = (int64_t)H * DV;
  float nxt = k0 < k1 ? part[(int64_t)k0 * stride + e] : 0.f;
  int pw_rows = -1;
  float pw = 1.f;
  for (int k = k0; k < k1; ++k) {
    const float local = nxt;
    if (k + 1 < k1) nxt = part[(int64_t)(k + 1) * stride + e];
    const int rws = chunk_rows[k];
    if (rws != pw_rows) {
      pw = powf(lam, (float)rws);
      pw_rows = rws;
    }
    part[(int64_t)k * stride + e] = carry;
    carry = pw * carry + local;
  }
  if (slot >= 0) state[(int64_t)slot * H * DV + se] = carry;
}

}  // namespace arks

using namespace arks;

extern "C" void arks_seq_lightning_combine(void* part, const void* decay,
                                           void* state, const void* chunk_off,
                                           const void* chunk_rows,
                                           const void* cu, const void* seq_lens,
                                           const void* slots, int S, int H,
                                           int D, int V, int transposed,
                                           hipStream_t stream) {
  if (S == 0) return;
  const int64_t n = (int64_t)H * D * V;
  hipLaunchKernelGGL(lightning_combine_kernel,
                     dim3((unsigned)((n + 255) / 256), S), dim3(256), 0, stream,
                     (float*)part, (const float*)decay, (float*)state,
                     (const int*)chunk_off, (const int*)chunk_rows,
                     (const int*)cu, (const int*)seq_lens, (const int*)slots, H,
                     D, V, transposed);
}

template <typename AT, int MODE>
static int launch_lightning(float* out, const void* q, const void* k,
                            const void* v, int64_t ldq, int64_t ldk,
                            int64_t ldv, const float* decay, float* state,
                            const int* cu, const int* seq_lens,
                            const int* slots, int S, int H, int D, int V,
                            const int64_t* positions, const float* freq,
                            int n_rot, int interleaved, float k_scale,
                            hipStream_t stream) {
  dim3 grid(S, H, (V + 63) / 64), block(64);
#define LL(DM)                                                                 \
  hipLaunchKernelGGL((lightning_scan_kernel<AT, DM, MODE>), grid, block, 0,    \
                     stream, out, (const AT*)q, (const AT*)k, (const AT*)v,    \
                     ldq, ldk, ldv, decay, state, cu, seq_lens, slots, H, D,   \
                     V, positions, freq, n_rot, interleaved, k_scale)
  if (D <= 16) LL(16);
  else if (D <= 32) LL(32);
  else if (D <= 64) LL(64);
  else if (D <= 128) LL(128);
  else if (D <= 256) LL(256);
  else return 1;
#undef LL
  return 0;
}

extern "C" int arks_seq_lightning_scan(
    void* out, const void* q, const void* k, const void* v, int64_t ldq,
    int64_t ldk, int64_t ldv, const void* decay, void* state, const void* cu,
    const void* seq_lens, const void* slots, int S, int H, int D, int V,
    int act_f32, int mode, const void* positions, const void* freq, int n_rot,
    int interleaved, float k_scale, hipStream_t stream) {
  if (S == 0) return 0;
  int rc = 0;
#define LS(MODE)                                                              \
  SEQ_DISPATCH_ACT(act_f32, (rc = launch_lightning<AT, MODE>(                 \
      (float*)out, q, k, v, ldq, ldk, ldv, (const float*)decay, (float*)state, \
      (const int*)cu, (const int*)seq_lens, (const int*)slots, S, H, D, V,    \
      (const int64_t*)positions, (const float*)freq, n_rot, interleaved,      \
      k_scale, stream)))
  if (mode == 0) LS(0);
  else LS(1);
#undef LS
  return rc;
}
