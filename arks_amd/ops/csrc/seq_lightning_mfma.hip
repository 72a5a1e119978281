// Lightning attention prefill on the matrix cores (bf16 rows, gfx950):
// the two scans of the chunk-parallel scheme (ops.scan_chunks) as 64-row
// block products, one workgroup of 4 waves per (chunk, head).
//
//   pass 1  part[d][v] = sum_j decay^(n-1-j) k_j[d] v_j[v]      (n rows)
//   pass 2  o_i = decay^(i+1) (q_i . S0) + sum_{j<=i} decay^(i-j) (q_i.k_j) v_j
//
// with S0 the chunk's start state left in `part` by lightning_combine.
// `part` holds each state TRANSPOSED ([v][d]): pass 2 then reads its state
// operand (k = d contiguous) straight from global memory, and the combine
// step between the passes is elementwise, so it does not care.
// q, k, v are silu'd (MODE 0), or q and k turned by their position and k
// scaled (MODE 1, see seq_lightning.hip), in fp32 on the way into LDS and
// rounded to bf16 for v_mfma_f32_16x16x32_bf16. Every fp32 quantity that meets a matrix
// operand — the decayed keys of pass 1, the decayed score matrix and the
// fp32 state of pass 2 — is split into a bf16 high and low part and
// multiplied twice, so decays, scores and state keep ~16 mantissa bits
// through the products; accumulation is fp32.
//
// Operand convention (as in attn_extend.hip): mfma(a, b) gives
// D[m][n] = sum_k a[m][k] b[n][k]; a lane holds row (lane % 16) and k =
// 8 (lane / 16) .. +7 of each 32-wide k step; the result lane holds column
// n = lane % 16, rows m = 4 (lane / 16) + r. So every operand sits in LDS
// with k contiguous: V, decayed K and the state are staged transposed.
#include "seq_common.h"

namespace arks {

struct LmRot {  // MODE 1 input transform
  const int64_t* positions;
  const float* freq;
  int n_rot, interleaved;
  float k_scale;
};

// Element d of head row `row` (bf16): silu (MODE 0) or position turn.
template <int MODE>
__device__ __forceinline__ float lm_load(const bf16* row, int d, int64_t t,
                                         const LmRot& rot) {
  const float x = bf16_bits_to_float(row[d]);
  if (MODE == 0) return silu_f(x);
  if (d >= 2 * rot.n_rot) return x;
  const int n = rot.n_rot;
  const int i = rot.interleaved ? d >> 1 : (d < n ? d : d - n);
  const bool first = rot.interleaved ? !(d & 1) : d < n;
  const int dp = rot.interleaved ? d ^ 1 : (first ? d + n : d - n);
  const float y = bf16_bits_to_float(row[dp]);
  float sn, cs;
  sincosf((float)rot.positions[t] * rot.freq[i], &sn, &cs);
  return first ? x * cs - y * sn : x * cs + y * sn;
}

// MODE 1 staging walks a head row in pairs so that one sine/cosine serves
// both dims of a pair (and q and k of the row): pair p < n_rot is a rotary
// pair, later pairs are two neighbouring plain dims.
__device__ __forceinline__ void lm_pair_dims(const LmRot& rot, int p, int& d0,
                                             int& d1) {
  if (p < rot.n_rot) {
    d0 = rot.interleaved ? 2 * p : p;
    d1 = rot.interleaved ? 2 * p + 1 : p + rot.n_rot;
  } else {
    d0 = 2 * p;
    d1 = 2 * p + 1;
  }
}

__device__ __forceinline__ void lm_turn(const bf16* row, int d0, int d1,
                                        float cs, float sn, float& x0,
                                        float& x1) {
  const float a = bf16_bits_to_float(row[d0]), b = bf16_bits_to_float(row[d1]);
  x0 = a * cs - b * sn;
  x1 = b * cs + a * sn;
}

typedef __attribute__((ext_vector_type(8))) __bf16 lm_bf16x8;
typedef __attribute__((ext_vector_type(4))) float lm_f32x4;

constexpr int LM_ROWS = 64;  // rows per chunk (ops.SCAN_CHUNK)
constexpr int LM_PAD = 8;    // bf16 elements of row padding in LDS

__device__ __forceinline__ lm_f32x4 lm_mfma(const bf16* a, const bf16* b,
                                            lm_f32x4 c) {
  ushort8 ua = *reinterpret_cast<const ushort8*>(a);
  ushort8 ub = *reinterpret_cast<const ushort8*>(b);
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
      *reinterpret_cast<lm_bf16x8*>(&ua), *reinterpret_cast<lm_bf16x8*>(&ub), c,
      0, 0, 0);
}

__device__ __forceinline__ lm_f32x4 lm_mfma_r(const bf16* a, ushort8 ub,
                                              lm_f32x4 c) {
  ushort8 ua = *reinterpret_cast<const ushort8*>(a);
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
      *reinterpret_cast<lm_bf16x8*>(&ua), *reinterpret_cast<lm_bf16x8*>(&ub), c,
      0, 0, 0);
}

__device__ __forceinline__ void split_bf16(float x, bf16& hi, bf16& lo) {
  hi = float_to_bf16_bits(x);
  lo = float_to_bf16_bits(x - bf16_bits_to_float(hi));
}

// decay^e for integer e >= 0 (0^0 = 1)
__device__ __forceinline__ float decay_pow(float log2_decay, int e) {
  return e == 0 ? 1.f : __builtin_amdgcn_exp2f(log2_decay * (float)e);
}

// ---- pass 1: end state of each chunk scanned from zero
template <int D, int V, int MODE>
__global__ __launch_bounds__(256) void lightning_state_mfma_kernel(
    float* __restrict__ part,  // [chunks, H, V, D] (transposed states)
    const bf16* __restrict__ k, const bf16* __restrict__ v, int64_t ldk,
    int64_t ldv, const float* __restrict__ decay, const int* __restrict__ cu,
    int H, LmRot rot) {
  constexpr int LK = LM_ROWS + LM_PAD;
  extern __shared__ __attribute__((aligned(16))) unsigned char lm_smem[];
  bf16* kt_hi = reinterpret_cast<bf16*>(lm_smem);  // [D][LK]
  bf16* kt_lo = kt_hi + D * LK;                    // [D][LK]
  bf16* vt = kt_lo + D * LK;                       // [V][LK]
  const int ch = blockIdx.x, h = blockIdx.y;
  const int row0 = cu[ch], n = cu[ch + 1] - row0;
  const float l2 = log2f(decay[h]);
  const int tid = threadIdx.x;
  if (MODE == 0) {
    for (int i = tid; i < LM_ROWS * D; i += 256) {
      const int j = i / D, d = i - j * D;
      float x = 0.f;
      if (j < n)
        x = lm_load<0>(k + (int64_t)(row0 + j) * ldk + (int64_t)h * D, d,
                       row0 + j, rot) * decay_pow(l2, n - 1 - j);
      split_bf16(x, kt_hi[d * LK + j], kt_lo[d * LK + j]);
    }
  } else {
    for (int i = tid; i < LM_ROWS * (D / 2); i += 256) {
      const int j = i / (D / 2), p = i - j * (D / 2);
      int d0, d1;
      lm_pair_dims(rot, p, d0, d1);
      float x0 = 0.f, x1 = 0.f;
      if (j < n) {
        float sn = 0.f, cs = 1.f;
        if (p < rot.n_rot)
          sincosf((float)rot.positions[row0 + j] * rot.freq[p], &sn, &cs);
        lm_turn(k + (int64_t)(row0 + j) * ldk + (int64_t)h * D, d0, d1, cs, sn,
                x0, x1);
        const float f = rot.k_scale * decay_pow(l2, n - 1 - j);
        x0 *= f;
        x1 *= f;
      }
      split_bf16(x0, kt_hi[d0 * LK + j], kt_lo[d0 * LK + j]);
      split_bf16(x1, kt_hi[d1 * LK + j], kt_lo[d1 * LK + j]);
    }
  }
  for (int i = tid; i < LM_ROWS * V; i += 256) {
    const int j = i / V, c = i - j * V;
    float x = 0.f;
    if (j < n) {
      x = bf16_bits_to_float(v[(int64_t)(row0 + j) * ldv + (int64_t)h * V + c]);
      if (MODE == 0) x = silu_f(x);
    }
    vt[c * LK + j] = float_to_bf16_bits(x);
  }
  __syncthreads();
  const int wave = tid / 64, lane = tid % 64, lq = lane % 16, la = lane / 16;
  constexpr int DT = D / 16, VT = V / 16;
  float* out = part + ((int64_t)ch * H + h) * D * V;
  for (int dt = wave; dt < DT; dt += 4) {
    lm_f32x4 acc[VT];
#pragma unroll
    for (int c = 0; c < VT; ++c) acc[c] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int st = 0; st < LM_ROWS / 32; ++st) {
      const int ko = st * 32 + 8 * la;
      const bf16* bh = kt_hi + (dt * 16 + lq) * LK + ko;
      const bf16* bl = kt_lo + (dt * 16 + lq) * LK + ko;
#pragma unroll
      for (int c = 0; c < VT; ++c) {
        const bf16* a = vt + (c * 16 + lq) * LK + ko;  // rows = value dims
        acc[c] = lm_mfma(a, bh, acc[c]);
        acc[c] = lm_mfma(a, bl, acc[c]);
      }
    }
    // result rows m = value dim, column n = key dim: out[v][d]
#pragma unroll
    for (int c = 0; c < VT; ++c)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        out[(int64_t)(c * 16 + 4 * la + r) * D + dt * 16 + lq] = acc[c][r];
  }
}

// ---- pass 2: outputs of each chunk from its start state
template <int D, int V, int MODE>
__global__ __launch_bounds__(256) void lightning_out_mfma_kernel(
    float* __restrict__ out,         // [T, H, V] fp32
    const float* __restrict__ part,  // [chunks, H, V, D] start states^T
    const bf16* __restrict__ q, const bf16* __restrict__ k,
    const bf16* __restrict__ v, int64_t ldq, int64_t ldk, int64_t ldv,
    const float* __restrict__ decay, const int* __restrict__ cu, int H,
    LmRot rot) {
  constexpr int LD = D + LM_PAD;
  constexpr int LK = LM_ROWS + LM_PAD;
  extern __shared__ __attribute__((aligned(16))) unsigned char lm_smem[];
  bf16* qs = reinterpret_cast<bf16*>(lm_smem);  // [64][LD]
  bf16* ks = qs + LM_ROWS * LD;                 // [64][LD]
  bf16* vt = ks + LM_ROWS * LD;                 // [V][LK]
  bf16* a_hi = vt + V * LK;                     // [64][LK]
  bf16* a_lo = a_hi + LM_ROWS * LK;             // [64][LK]
  const int ch = blockIdx.x, h = blockIdx.y;
  const int row0 = cu[ch], n = cu[ch + 1] - row0;
  const float l2 = log2f(decay[h]);
  const int tid = threadIdx.x;
  if (MODE == 0) {
    for (int i = tid; i < LM_ROWS * D; i += 256) {
      const int j = i / D, d = i - j * D;
      float xq = 0.f, xk = 0.f;
      if (j < n) {
        xq = lm_load<0>(q + (int64_t)(row0 + j) * ldq + (int64_t)h * D, d,
                        row0 + j, rot);
        xk = lm_load<0>(k + (int64_t)(row0 + j) * ldk + (int64_t)h * D, d,
                        row0 + j, rot);
      }
      qs[j * LD + d] = float_to_bf16_bits(xq);
      ks[j * LD + d] = float_to_bf16_bits(xk);
    }
  } else {
    for (int i = tid; i < LM_ROWS * (D / 2); i += 256) {
      const int j = i / (D / 2), p = i - j * (D / 2);
      int d0, d1;
      lm_pair_dims(rot, p, d0, d1);
      float q0 = 0.f, q1 = 0.f, k0 = 0.f, k1 = 0.f;
      if (j < n) {
        float sn = 0.f, cs = 1.f;
        if (p < rot.n_rot)
          sincosf((float)rot.positions[row0 + j] * rot.freq[p], &sn, &cs);
        lm_turn(q + (int64_t)(row0 + j) * ldq + (int64_t)h * D, d0, d1, cs, sn,
                q0, q1);
        lm_turn(k + (int64_t)(row0 + j) * ldk + (int64_t)h * D, d0, d1, cs, sn,
                k0, k1);
        k0 *= rot.k_scale;
        k1 *= rot.k_scale;
      }
      qs[j * LD + d0] = float_to_bf16_bits(q0);
      qs[j * LD + d1] = float_to_bf16_bits(q1);
      ks[j * LD + d0] = float_to_bf16_bits(k0);
      ks[j * LD + d1] = float_to_bf16_bits(k1);
    }
  }
  for (int i = tid; i < LM_ROWS * V; i += 256) {
    const int j = i / V, c = i - j * V;
    float x = 0.f;
    if (j < n) {
      x = bf16_bits_to_float(v[(int64_t)(row0 + j) * ldv + (int64_t)h * V + c]);
      if (MODE == 0) x = silu_f(x);
    }
    vt[c * LK + j] = float_to_bf16_bits(x);
  }
  const float* sp = part + ((int64_t)ch * H + h) * D * V;  // [V][D]
  __syncthreads();
  const int wave = tid / 64, lane = tid % 64, lq = lane % 16, la = lane / 16;
  // scores of this wave's 16 rows against all 64 keys, decayed and masked,
  // into a_hi/a_lo[i][j] (each wave writes only its own rows)
  const int irow = wave * 16 + lq;  // the row this lane's score column is
#pragma unroll
  for (int jt = 0; jt < LM_ROWS / 16; ++jt) {
    lm_f32x4 sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int st = 0; st < D / 32; ++st) {
      const int ko = st * 32 + 8 * la;
      sc = lm_mfma(ks + (jt * 16 + lq) * LD + ko, qs + irow * LD + ko, sc);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int j = jt * 16 + 4 * la + r;
      const float w = (j <= irow && irow < n) ? sc[r] * decay_pow(l2, irow - j) : 0.f;
      split_bf16(w, a_hi[irow * LK + j], a_lo[irow * LK + j]);
    }
  }
  __syncthreads();
  constexpr int VT = V / 16;
  lm_f32x4 acc[VT], acs[VT];
#pragma unroll
  for (int c = 0; c < VT; ++c) {
    acc[c] = {0.f, 0.f, 0.f, 0.f};
    acs[c] = {0.f, 0.f, 0.f, 0.f};
  }
  const int arow = wave * 16 + lq;  // A-operand row of this lane
#pragma unroll
  for (int st = 0; st < LM_ROWS / 32; ++st) {
    const int ko = st * 32 + 8 * la;
#pragma unroll
    for (int c = 0; c < VT; ++c) {
      const bf16* b = vt + (c * 16 + lq) * LK + ko;
      acc[c] = lm_mfma(a_hi + arow * LK + ko, b, acc[c]);
      acc[c] = lm_mfma(a_lo + arow * LK + ko, b, acc[c]);
    }
  }
#pragma unroll
  for (int st = 0; st < D / 32; ++st) {
    const int ko = st * 32 + 8 * la;
#pragma unroll
    for (int c = 0; c < VT; ++c) {
      // 8 consecutive key dims of state row v = 16 c + lq, fp32 -> hi + lo
      const float* sr = sp + (int64_t)(c * 16 + lq) * D + ko;
      const float4v s0 = *reinterpret_cast<const float4v*>(sr);
      const float4v s1 = *reinterpret_cast<const float4v*>(sr + 4);
      ushort8 bh, bl;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        bf16 h0, l0, h1, l1;
        split_bf16(s0[e], h0, l0);
        split_bf16(s1[e], h1, l1);
        bh[e] = h0; bl[e] = l0; bh[4 + e] = h1; bl[4 + e] = l1;
      }
      acs[c] = lm_mfma_r(qs + arow * LD + ko, bh, acs[c]);
      acs[c] = lm_mfma_r(qs + arow * LD + ko, bl, acs[c]);
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int i = wave * 16 + 4 * la + r;
    if (i >= n) continue;
    const float carry = decay_pow(l2, i + 1);
    float* orow = out + ((int64_t)(row0 + i) * H + h) * V;
#pragma unroll
    for (int c = 0; c < VT; ++c) orow[c * 16 + lq] = acc[c][r] + carry * acs[c][r];
  }
}

}  // namespace arks

using namespace arks;

template <int D, int V, int MODE>
static void launch_lm(float* out, float* part, const void* q, const void* k,
                      const void* v, int64_t ldq, int64_t ldk, int64_t ldv,
                      const float* decay, const int* cu, int chunks, int H,
                      int pass, LmRot rot, hipStream_t stream) {
  constexpr int LD = D + LM_PAD, LK = LM_ROWS + LM_PAD;
  dim3 grid(chunks, H), block(256);
  if (pass == 1) {
    constexpr int lds = (2 * D * LK + V * LK) * 2;
    static bool set = false;
    if (!set) {
      (void)hipFuncSetAttribute(
          reinterpret_cast<const void*>(lightning_state_mfma_kernel<D, V, MODE>),
          hipFuncAttributeMaxDynamicSharedMemorySize, lds);
      set = true;
    }
    hipLaunchKernelGGL((lightning_state_mfma_kernel<D, V, MODE>), grid, block, lds,
                       stream, part, (const bf16*)k, (const bf16*)v, ldk, ldv,
                       decay, cu, H, rot);
  } else {
    constexpr int lds = (2 * LM_ROWS * LD + V * LK + 2 * LM_ROWS * LK) * 2;
    static bool set = false;
    if (!set) {
      (void)hipFuncSetAttribute(
          reinterpret_cast<const void*>(lightning_out_mfma_kernel<D, V, MODE>),
          hipFuncAttributeMaxDynamicSharedMemorySize, lds);
      set = true;
    }
    hipLaunchKernelGGL((lightning_out_mfma_kernel<D, V, MODE>), grid, block, lds,
                       stream, out, part, (const bf16*)q, (const bf16*)k,
                       (const bf16*)v, ldq, ldk, ldv, decay, cu, H, rot);
  }
}

// pass 1: part <- chunk end states; pass 2: out <- rows, part = start states.
// Returns 1 when no kernel is built for (D, V).
extern "C" int arks_seq_lightning_mfma(void* out, void* part, const void* q,
                                       const void* k, const void* v,
                                       int64_t ldq, int64_t ldk, int64_t ldv,
                                       const void* decay, const void* cu,
                                       int chunks, int H, int D, int V,
                                       int pass, int mode,
                                       const void* positions, const void* freq,
                                       int n_rot, int interleaved,
                                       float k_scale, hipStream_t stream) {
  if (chunks == 0) return 0;
  const LmRot rot{(const int64_t*)positions, (const float*)freq, n_rot,
                  interleaved, k_scale};
#define LM(DD, VV)                                                            \
  if (D == DD && V == VV) {                                                   \
    if (mode == 0)                                                            \
      launch_lm<DD, VV, 0>((float*)out, (float*)part, q, k, v, ldq, ldk, ldv, \
                           (const float*)decay, (const int*)cu, chunks, H,    \
                           pass, rot, stream);                                \
    else                                                                      \
      launch_lm<DD, VV, 1>((float*)out, (float*)part, q, k, v, ldq, ldk, ldv, \
                           (const float*)decay, (const int*)cu, chunks, H,    \
                           pass, rot, stream);                                \
    return 0;                                                                 \
  }
  LM(32, 32)
  LM(64, 64)
  LM(128, 128)
  LM(64, 128)
  LM(128, 64)
  LM(64, 32)
  LM(128, 32)
#undef LM
  return 1;
}
