// Mamba1 mixer kernels: the short causal depthwise convolution (+ silu) with
// its per-sequence history, and the selective scan
//   S[c,n] <- exp(dt_c A[c,n]) S[c,n] + dt_c u_c B_n
//   y_c = sum_n S[c,n] C_n + D_c u_c,   out = y * silu(z)
// with dt = softplus(W_dt dt_raw + b) computed here in fp32, S fp32 in a
// slot-addressed state tensor.
#include "seq_common.h"

namespace arks {

constexpr int CONV_MAX_HIST = 8;  // taps - 1

// One block per row, threads over channels. Inputs before the step's first
// row come from the sequence's stored history (zeros at position 0). The
// history is replaced by conv_state_update_kernel in a later launch, so
// every reader here sees the old one.
template <typename AT>
__global__ __launch_bounds__(256) void causal_conv_silu_kernel(
    AT* __restrict__ out, const AT* __restrict__ x, int64_t ldx,
    const float* __restrict__ w, const float* __restrict__ bias,
    const float* __restrict__ state, const int* __restrict__ cu,
    const int* __restrict__ seq_lens, const int* __restrict__ slots,
    const int* __restrict__ token_seq, int C, int taps) {
  const int t = blockIdx.x;
  const SeqRow r = seq_row(t, token_seq, cu, seq_lens, slots);
  const int i = t - r.first_row;
  const bool has_state = r.start > 0 && r.slot >= 0;
  const float* hist = state + (int64_t)(r.slot < 0 ? 0 : r.slot) * (taps - 1) * C;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < C; c += gridDim.y * 256) {
    float acc = bias[c];
    for (int j = 0; j < taps; ++j) {
      const int src = i - (taps - 1 - j);
      float xv;
      if (src >= 0)
        xv = Act<AT>::ld(x + (int64_t)(r.first_row + src) * ldx + c);
      else
        xv = has_state ? hist[(int64_t)(src + taps - 1) * C + c] : 0.f;
      acc += w[(int64_t)c * taps + j] * xv;
    }
    Act<AT>::st(out + (int64_t)t * C + c, silu_f(acc));
  }
}

// bf16 rows, 8 channels per thread and CONV_RPT consecutive rows per block:
// 16-byte loads of each tap's row, the conv taps of the thread's channels
// held in registers across the rows (w_t [taps, C] is a transposed copy of
// the weights so that they load as two float4 per tap).
constexpr int CONV_RPT = 8;
constexpr int CONV_MAX_TAPS = CONV_MAX_HIST + 1;

__global__ __launch_bounds__(256) void causal_conv_silu_vec8_kernel(
    bf16* __restrict__ out, const bf16* __restrict__ x, int64_t ldx,
    const float* __restrict__ w_t, const float* __restrict__ bias,
    const float* __restrict__ state, const int* __restrict__ cu,
    const int* __restrict__ seq_lens, const int* __restrict__ slots,
    const int* __restrict__ token_seq, int T, int C, int taps) {
  const int c = (blockIdx.y * 256 + threadIdx.x) * 8;
  if (c >= C) return;
  float wv[CONV_MAX_TAPS][8], bv[8];
  {
    const float4v b0 = *reinterpret_cast<const float4v*>(bias + c);
    const float4v b1 = *reinterpret_cast<const float4v*>(bias + c + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) { bv[e] = b0[e]; bv[4 + e] = b1[e]; }
  }
#pragma unroll
  for (int j = 0; j < CONV_MAX_TAPS; ++j) {
    if (j < taps) {
      const float4v w0 = *reinterpret_cast<const float4v*>(w_t + (int64_t)j * C + c);
      const float4v w1 = *reinterpret_cast<const float4v*>(w_t + (int64_t)j * C + c + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { wv[j][e] = w0[e]; wv[j][4 + e] = w1[e]; }
    }
  }
  const int t_end = min(T, (int)(blockIdx.x + 1) * CONV_RPT);
  for (int t = blockIdx.x * CONV_RPT; t < t_end; ++t) {
    const SeqRow r = seq_row(t, token_seq, cu, seq_lens, slots);
    const int i = t - r.first_row;
    const bool has_state = r.start > 0 && r.slot >= 0;
    const float* hist =
        state + (int64_t)(r.slot < 0 ? 0 : r.slot) * (taps - 1) * C;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = bv[e];
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) {
      if (j < taps) {
        const int src = i - (taps - 1 - j);
        float xv[8];
        bool have = true;
        if (src >= 0) {
          const ushort8 v = *reinterpret_cast<const ushort8*>(
              x + (int64_t)(r.first_row + src) * ldx + c);
#pragma unroll
          for (int e = 0; e < 8; ++e) xv[e] = bf16_bits_to_float(v[e]);
        } else if (has_state) {
          const float* hp = hist + (int64_t)(src + taps - 1) * C + c;
          const float4v h0 = *reinterpret_cast<const float4v*>(hp);
          const float4v h1 = *reinterpret_cast<const float4v*>(hp + 4);
#pragma unroll
          for (int e = 0; e < 4; ++e) { xv[e] = h0[e]; xv[4 + e] = h1[e]; }
        } else {
          have = false;
        }
        if (have) {
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[e] += wv[j][e] * xv[e];
        }
      }
    }
    ushort8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = float_to_bf16_bits(silu_f(acc[e]));
    *reinterpret_cast<ushort8*>(out + (int64_t)t * C + c) = o;
  }
}

// New history of a sequence = the last taps-1 inputs after this step: rows
// of this step where there are enough, older history shifted up otherwise.
// One thread per (sequence, channel) reads all it needs before it writes.
template <typename AT>
__global__ __launch_bounds__(256) void conv_state_update_kernel(
    float* __restrict__ state, const AT* __restrict__ x, int64_t ldx,
    const int* __restrict__ cu, const int* __restrict__ seq_lens,
    const int* __restrict__ slots, int C, int taps) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  const int a = cu[s], rows = cu[s + 1] - a;
  const int slot = slots[s];
  if (c >= C || rows == 0 || slot < 0) return;
  const int start = seq_lens[s] - rows;
  const int nh = taps - 1;
  float* hist = state + (int64_t)slot * nh * C + c;
  float nv[CONV_MAX_HIST];
#pragma unroll
  for (int i = 0; i < CONV_MAX_HIST; ++i) {
    if (i < nh) {
      const int src = rows - nh + i;  // index into this step's rows
      if (src >= 0)
        nv[i] = Act<AT>::ld(x + (int64_t)(a + src) * ldx + c);
      else
        nv[i] = start > 0 ? hist[(int64_t)(src + nh) * C] : 0.f;
    }
  }
#pragma unroll
  for (int i = 0; i < CONV_MAX_HIST; ++i)
    if (i < nh) hist[(int64_t)i * C] = nv[i];
}

// Selective scan: 16 lanes per channel (4 channels per wave), lane ln owns
// states n = ln + 16 i. Rows are walked in order; the output sum is reduced
// over the 16 lanes. dt's pre-activation either comes from a GEMM (dt_pre,
// fp32 [T, C]) or is projected here from dt_raw. dsum (optional, [S, C])
// receives each sequence's sum of dt — what the chunk-parallel prefill
// needs to carry a state across a chunk: prod_t exp(dt_t A) = exp(A dsum).
template <typename AT, int NPT>
__global__ __launch_bounds__(64) void selective_scan_kernel(
    AT* __restrict__ out, const AT* __restrict__ u, const AT* __restrict__ dbc,
    int64_t ldd, const AT* __restrict__ z, int64_t ldz,
    const float* __restrict__ dt_w, const float* __restrict__ dt_b,
    const float* __restrict__ A, const float* __restrict__ Dp,
    float* __restrict__ state, const int* __restrict__ cu,
    const int* __restrict__ seq_lens, const int* __restrict__ slots, int C,
    int N, int R, const float* __restrict__ dt_pre, float* __restrict__ dsum) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * 4 + threadIdx.x / 16;
  const int ln = threadIdx.x % 16;
  const int a = cu[s], rows = cu[s + 1] - a;
  if (rows == 0) return;
  const bool live = c < C;
  const int cc = live ? c : C - 1;  // keep the whole wave in the shuffles
  const int start = seq_lens[s] - rows;
  const int slot = slots[s];
  const bool has_state = start > 0 && slot >= 0;
  float* sp = state + ((int64_t)(slot < 0 ? 0 : slot) * C + cc) * N;
  float S[NPT], Av[NPT];
#pragma unroll
  for (int i = 0; i < NPT; ++i) {
    const int n = ln + 16 * i;
    S[i] = (has_state && n < N) ? sp[n] : 0.f;
    Av[i] = n < N ? A[(int64_t)cc * N + n] : 0.f;
  }
  const float dtb = dt_b[cc], dd = Dp[cc];
  const float* wr = dt_w + (int64_t)cc * R;
  float dts = 0.f;
  for (int r = 0; r < rows; ++r) {
    const int t = a + r;
    const AT* drow = dbc + (int64_t)t * ldd;
    float dtp;
    if (dt_pre) {
      dtp = dt_pre[(int64_t)t * C + cc];
    } else {
      dtp = 0.f;
      for (int j = ln; j < R; j += 16) dtp += wr[j] * Act<AT>::ld(drow + j);
      dtp = group16_reduce_sum(dtp);
    }
    const float dt = softplus_f(dtp + dtb);
    dts += dt;
    const float xv = Act<AT>::ld(u + (int64_t)t * C + cc);
    const float dx = dt * xv;
    float y = 0.f;
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
      const int n = ln + 16 * i;
      if (n < N) {
        const float Bn = Act<AT>::ld(drow + R + n);
        const float Cn = Act<AT>::ld(drow + R + N + n);
        S[i] = expf(dt * Av[i]) * S[i] + dx * Bn;
        y += S[i] * Cn;
      }
    }
    y = group16_reduce_sum(y) + dd * xv;
    if (ln == 0 && live) {
      const float zv = Act<AT>::ld(z + (int64_t)t * ldz + c);
      Act<AT>::st(out + (int64_t)t * C + c, y * silu_f(zv));
    }
  }
  if (slot >= 0 && live) {
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
      const int n = ln + 16 * i;
      if (n < N) sp[n] = S[i];
    }
  }
  if (dsum && ln == 0 && live) dsum[(int64_t)s * C + c] = dts;
}

// Selective scan for small state sizes with dt from a GEMM: one LANE per
// channel, its N states in registers; a block of 256 threads covers 256
// consecutive channels of one sequence (or chunk). Row operands u / dt_pre
// / z are read coalesced across channels; B and C of the rows — the same
// for every channel — are staged in LDS as floats, SCAN_ROWS rows at a
// time, and read back as broadcasts. The sum over states stays inside the
// lane: no shuffles, 16x fewer waves than the lane-split kernel above for
// N = 16. bf16 serving folds log2(e) into A and uses the hardware exp2;
// float rows keep the precise expf. WITH_Y = false is the first pass of the
// chunk-parallel prefill: only the end state and the sum of dt are needed.
// Same arguments and state handling as selective_scan_kernel.
constexpr int SCAN_ROWS = 32;

template <typename AT, int NMAX, bool WITH_Y>
__global__ __launch_bounds__(256) void selective_scan_lane_kernel(
    AT* __restrict__ out, const AT* __restrict__ u, const AT* __restrict__ dbc,
    int64_t ldd, const AT* __restrict__ z, int64_t ldz,
    const float* __restrict__ dt_b, const float* __restrict__ A,
    const float* __restrict__ Dp, float* __restrict__ state,
    const int* __restrict__ cu, const int* __restrict__ seq_lens,
    const int* __restrict__ slots, int C, int N, int R,
    const float* __restrict__ dt_pre, float* __restrict__ dsum) {
  constexpr bool FAST = sizeof(AT) == 2;
  __shared__ float bc_s[SCAN_ROWS][2 * NMAX];
  const int s = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int a = cu[s], rows = cu[s + 1] - a;
  if (rows == 0) return;
  const bool live = c < C;
  const int cc = live ? c : C - 1;
  const int start = seq_lens[s] - rows;
  const int slot = slots[s];
  const bool has_state = start > 0 && slot >= 0;
  float* sp = state + ((int64_t)(slot < 0 ? 0 : slot) * C + cc) * N;
  float S[NMAX], Av[NMAX];
#pragma unroll
  for (int n = 0; n < NMAX; ++n) {
    S[n] = (has_state && n < N) ? sp[n] : 0.f;
    Av[n] = n < N ? A[(int64_t)cc * N + n] : 0.f;
    if (FAST) Av[n] *= 1.4426950408889634f;
  }
  const float dtb = dt_b[cc], dd = Dp[cc];
  float dts = 0.f;
  for (int r0 = 0; r0 < rows; r0 += SCAN_ROWS) {
    const int nr = min(SCAN_ROWS, rows - r0);
    __syncthreads();  // the previous tile's readers are done
    for (int i = threadIdx.x; i < nr * 2 * N; i += 256) {
      const int rr = i / (2 * N), col = i - rr * 2 * N;
      bc_s[rr][col < N ? col : NMAX + (col - N)] =
          Act<AT>::ld(dbc + (int64_t)(a + r0 + rr) * ldd + R + col);
    }
    __syncthreads();
    for (int rr = 0; rr < nr; ++rr) {
      const int t = a + r0 + rr;
      const float dt = softplus_f(dt_pre[(int64_t)t * C + cc] + dtb);
      const float xv = Act<AT>::ld(u + (int64_t)t * C + cc);
      dts += dt;
      const float dx = dt * xv;
      float y = 0.f;
#pragma unroll
      for (int n = 0; n < NMAX; ++n) {
        if (n < N) {
          const float e = FAST ? __builtin_amdgcn_exp2f(dt * Av[n])
                               : expf(dt * Av[n]);
          S[n] = e * S[n] + dx * bc_s[rr][n];
          if (WITH_Y) y += S[n] * bc_s[rr][NMAX + n];
        }
      }
      if (WITH_Y && live) {
        const float zv = Act<AT>::ld(z + (int64_t)t * ldz + cc);
        Act<AT>::st(out + (int64_t)t * C + c, (y + dd * xv) * silu_f(zv));
      }
    }
  }
  if (slot >= 0 && live) {
#pragma unroll
    for (int n = 0; n < NMAX; ++n)
      if (n < N) sp[n] = S[n];
  }
  if (dsum && live) dsum[(int64_t)s * C + c] = dts;
}

// Chunk-parallel prefill, middle step. Each sequence's rows were cut into
// chunks and scanned from zero state: part[k] holds chunk k's end state,
// dsum[k] its sum of dt. Walk a sequence's chunks in order, one thread per
// (channel, state): part[k] is replaced by the state at the START of chunk
// k (what the final pass scans from) and the sequence's slot receives the
// state after its last row.
__global__ __launch_bounds__(256) void scan_combine_kernel(
    float* __restrict__ part, const float* __restrict__ dsum,
    const float* __restrict__ A, float* __restrict__ state,
    const int* __restrict__ chunk_off, const int* __restrict__ cu,
    const int* __restrict__ seq_lens, const int* __restrict__ slots, int C,
    int N) {
  const int s = blockIdx.y;
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= (int64_t)C * N) return;
  const int c = (int)(e / N);
  const int rows = cu[s + 1] - cu[s];
  if (rows == 0) return;
  const int start = seq_lens[s] - rows;
  const int slot = slots[s];
  const float a = A[e];
  float carry = (start > 0 && slot >= 0) ? state[(int64_t)slot * C * N + e] : 0.f;
  for (int k = chunk_off[s]; k < chunk_off[s + 1]; ++k) {
    float* p = part + (int64_t)k * C * N + e;
    const float local = *p;
    *p = carry;
    carry = expf(a * dsum[(int64_t)k * C + c]) * carry + local;
  }
  if (slot >= 0) state[(int64_t)slot * C * N + e] = carry;
}

}  // namespace arks

using namespace arks;

extern "C" int arks_seq_causal_conv_silu(
    void* out, const void* x, int64_t ldx, const void* w, const void* w_t,
    const void* bias, void* state, const void* cu, const void* seq_lens,
    const void* slots, const void* token_seq, int T, int S, int C, int taps,
    int act_f32, hipStream_t stream) {
  if (taps - 1 > CONV_MAX_HIST || taps < 1) return 1;
  if (T == 0) return 0;
  const int cb = (C + 255) / 256;
  const bool vec8 = !act_f32 && w_t && C % 8 == 0 && ldx % 8 == 0 &&
                    ((uintptr_t)x % 16) == 0;
  SEQ_DISPATCH_ACT(act_f32, {
    if (vec8)
      hipLaunchKernelGGL(causal_conv_silu_vec8_kernel,
                         dim3((T + CONV_RPT - 1) / CONV_RPT,
                              (C / 8 + 255) / 256),
                         dim3(256), 0, stream, (bf16*)out, (const bf16*)x, ldx,
                         (const float*)w_t, (const float*)bias,
                         (const float*)state, (const int*)cu,
                         (const int*)seq_lens, (const int*)slots,
                         (const int*)token_seq, T, C, taps);
    else
    hipLaunchKernelGGL((causal_conv_silu_kernel<AT>), dim3(T, cb), dim3(256), 0,
                       stream, (AT*)out, (const AT*)x, ldx, (const float*)w,
                       (const float*)bias, (const float*)state, (const int*)cu,
                       (const int*)seq_lens, (const int*)slots,
                       (const int*)token_seq, C, taps);
    if (taps > 1)
      hipLaunchKernelGGL((conv_state_update_kernel<AT>), dim3(S, cb), dim3(256),
                         0, stream, (float*)state, (const AT*)x, ldx,
                         (const int*)cu, (const int*)seq_lens,
                         (const int*)slots, C, taps);
  });
  return 0;
}

template <typename AT>
static int launch_scan(void* out, const void* u, const void* dbc, int64_t ldd,
                       const void* z, int64_t ldz, const float* dt_w,
                       const float* dt_b, const float* A, const float* Dp,
                       float* state, const int* cu, const int* seq_lens,
                       const int* slots, int S, int C, int N, int R,
                       const float* dt_pre, float* dsum, hipStream_t stream) {
  if (dt_pre && N <= 64) {
    dim3 lgrid((C + 255) / 256, S);
    const bool with_y = out != nullptr;
#define SL(NM)                                                                \
  do {                                                                        \
    if (with_y)                                                               \
      hipLaunchKernelGGL((selective_scan_lane_kernel<AT, NM, true>), lgrid,   \
                         dim3(256), 0, stream, (AT*)out, (const AT*)u,        \
                         (const AT*)dbc, ldd, (const AT*)z, ldz, dt_b, A, Dp, \
                         state, cu, seq_lens, slots, C, N, R, dt_pre, dsum);  \
    else                                                                      \
      hipLaunchKernelGGL((selective_scan_lane_kernel<AT, NM, false>), lgrid,  \
                         dim3(256), 0, stream, (AT*)out, (const AT*)u,        \
                         (const AT*)dbc, ldd, (const AT*)z, ldz, dt_b, A, Dp, \
                         state, cu, seq_lens, slots, C, N, R, dt_pre, dsum);  \
  } while (0)
    if (N <= 8) SL(8);
    else if (N <= 16) SL(16);
    else if (N <= 32) SL(32);
    else SL(64);
#undef SL
    return 0;
  }
  dim3 grid((C + 3) / 4, S), block(64);
#define SS(NP)                                                                \
  hipLaunchKernelGGL((selective_scan_kernel<AT, NP>), grid, block, 0, stream, \
                     (AT*)out, (const AT*)u, (const AT*)dbc, ldd,             \
                     (const AT*)z, ldz, dt_w, dt_b, A, Dp, state, cu,         \
                     seq_lens, slots, C, N, R, dt_pre, dsum)
  if (N <= 16) SS(1);
  else if (N <= 32) SS(2);
  else if (N <= 64) SS(4);
  else if (N <= 128) SS(8);
  else if (N <= 256) SS(16);
  else return 1;
#undef SS
  return 0;
}

extern "C" int arks_seq_selective_scan(
    void* out, const void* u, const void* dbc, int64_t ldd, const void* z,
    int64_t ldz, const void* dt_w, const void* dt_b, const void* A,
    const void* Dp, void* state, const void* cu, const void* seq_lens,
    const void* slots, int S, int C, int N, int R, const void* dt_pre,
    void* dsum, int act_f32, hipStream_t stream) {
  if (S == 0) return 0;
  int rc = 0;
  SEQ_DISPATCH_ACT(act_f32, rc = launch_scan<AT>(
      out, u, dbc, ldd, z, ldz, (const float*)dt_w, (const float*)dt_b,
      (const float*)A, (const float*)Dp, (float*)state, (const int*)cu,
      (const int*)seq_lens, (const int*)slots, S, C, N, R,
      (const float*)dt_pre, (float*)dsum, stream));
  return rc;
}

extern "C" void arks_seq_scan_combine(void* part, const void* dsum,
                                      const void* A, void* state,
                                      const void* chunk_off, const void* cu,
                                      const void* seq_lens, const void* slots,
                                      int S, int C, int N,
                                      hipStream_t stream) {
  if (S == 0) return;
  const int64_t n = (int64_t)C * N;
  hipLaunchKernelGGL(scan_combine_kernel, dim3((unsigned)((n + 255) / 256), S),
                     dim3(256), 0, stream, (float*)part, (const float*)dsum,
                     (const float*)A, (float*)state, (const int*)chunk_off,
                     (const int*)cu, (const int*)seq_lens, (const int*)slots,
                     C, N);
}
