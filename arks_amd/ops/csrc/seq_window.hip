// Sliding-window attention with pooled blocks (arks_amd/models/mixers.py
// WindowPoolAttention), general kernels: any head sizes, bf16 or float rows
// and pages, fp32 arithmetic.
//
// The row at position i sees the keys j with 0 <= i - j < window and, in the
// same softmax, one pooled key/value for every block b of `pool` positions
// with b * pool + pool - 1 <= i - window. Pooled entries are the fp32 mean of
// the block's keys (values) as the pages hold them, written once when the
// block's last position is written: block b lives in the page of its first
// position p0 = b * pool, entry (p0 % block_size) / pool of the pooled caches
// [pages, G, spp, D|V].
#include "seq_common.h"

namespace arks {

// One block per row: the row's keys and values to their page.
template <typename AT>
__global__ __launch_bounds__(256) void kv_write_kernel(
    const AT* __restrict__ k, const AT* __restrict__ v, int64_t ldk,
    int64_t ldv, AT* __restrict__ k_cache, AT* __restrict__ v_cache,
    const int64_t* __restrict__ slot_mapping, int G, int D, int V, int bs) {
  const int t = blockIdx.x;
  const int64_t slot = slot_mapping[t];
  if (slot < 0) return;
  const int64_t page = slot / bs;
  const int off = (int)(slot % bs);
  for (int e = threadIdx.x; e < G * D; e += 256) {
    const int g = e / D, d = e - g * D;
    k_cache[((page * G + g) * bs + off) * D + d] = k[(int64_t)t * ldk + e];
  }
  for (int e = threadIdx.x; e < G * V; e += 256) {
    const int g = e / V, d = e - g * V;
    v_cache[((page * G + g) * bs + off) * V + d] = v[(int64_t)t * ldv + e];
  }
}

// bf16 rows whose heads are whole 16-byte pieces: one piece per thread.
__global__ __launch_bounds__(256) void kv_write_vec_kernel(
    const bf16* __restrict__ k, const bf16* __restrict__ v, int64_t ldk,
    int64_t ldv, bf16* __restrict__ k_cache, bf16* __restrict__ v_cache,
    const int64_t* __restrict__ slot_mapping, int G, int D, int V, int bs) {
  const int t = blockIdx.x;
  const int64_t slot = slot_mapping[t];
  if (slot < 0) return;
  const int64_t page = slot / bs;
  const int off = (int)(slot % bs);
  const int nk = G * D / 8, nv = G * V / 8;
  for (int i = threadIdx.x; i < nk + nv; i += 256) {
    const bool is_k = i < nk;
    const int e = (is_k ? i : i - nk) * 8;
    const int W = is_k ? D : V;
    const int g = e / W, d = e - g * W;
    const ushort8 u = *reinterpret_cast<const ushort8*>(
        (is_k ? k + (int64_t)t * ldk : v + (int64_t)t * ldv) + e);
    *reinterpret_cast<ushort8*>((is_k ? k_cache : v_cache) +
                                ((page * G + g) * bs + off) * W + d) = u;
  }
}

// One block per (64 rows, kv head): the rows whose position ends a block are
// listed first (one in `pool` of a prompt's rows), then the block's waves
// share them, lanes over the key and value dims. Runs after kv_write_kernel
// on the same stream, so it sees this step's rows.
template <typename AT>
__global__ __launch_bounds__(256) void kv_pool_kernel(
    const AT* __restrict__ k_cache, const AT* __restrict__ v_cache,
    AT* __restrict__ kp_cache, AT* __restrict__ vp_cache,
    const int64_t* __restrict__ slot_mapping,
    const int64_t* __restrict__ positions, const int* __restrict__ block_tables,
    const int* __restrict__ token_seq, int T, int max_blocks, int G, int D,
    int V, int bs, int pool, int spp) {
  __shared__ int list_s[64];
  __shared__ int count_s;
  const int g = blockIdx.y, tid = threadIdx.x;
  if (tid == 0) count_s = 0;
  __syncthreads();
  if (tid < 64) {
    const int t = blockIdx.x * 64 + tid;
    if (t < T && slot_mapping[t] >= 0 && (positions[t] + 1) % pool == 0)
      list_s[atomicAdd(&count_s, 1)] = t;
  }
  __syncthreads();
  const int wave = tid / 64, lane = tid % 64;
  for (int i = wave; i < count_s; i += 4) {
    const int t = list_s[i];
    const int* bt = block_tables + (int64_t)token_seq[t] * max_blocks;
    const int64_t p0 = positions[t] + 1 - pool;
    const int64_t page0 = bt[p0 / bs];
    const int e = (int)((p0 % bs) / pool);
    for (int d = lane; d < D + V; d += 64) {
      const bool is_k = d < D;
      const int dd = is_k ? d : d - D;
      const int W = is_k ? D : V;
      const AT* cache = is_k ? k_cache : v_cache;
      float acc = 0.f;
      for (int j = 0; j < pool; ++j) {
        const int64_t pos = p0 + j;
        const int64_t page = bt[pos / bs];
        acc += Act<AT>::ld(cache + ((page * G + g) * bs + pos % bs) * W + dd);
      }
      AT* dst = (is_k ? kp_cache : vp_cache) + ((page0 * G + g) * spp + e) * W + dd;
      Act<AT>::st(dst, acc / (float)pool);
    }
  }
}

// bf16 pages whose key + value dims make NC = (D + V) / 8 16-byte pieces with
// 64 % NC == 0: lane = (piece, position group); every lane sums its group's
// positions of its piece, the groups meet through shuffles.
__global__ __launch_bounds__(256) void kv_pool_vec_kernel(
    const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
    bf16* __restrict__ kp_cache, bf16* __restrict__ vp_cache,
    const int64_t* __restrict__ slot_mapping,
    const int64_t* __restrict__ positions, const int* __restrict__ block_tables,
    const int* __restrict__ token_seq, int T, int max_blocks, int G, int D,
    int V, int bs, int pool, int spp) {
  __shared__ int list_s[64];
  __shared__ int count_s;
  const int g = blockIdx.y, tid = threadIdx.x;
  if (tid == 0) count_s = 0;
  __syncthreads();
  if (tid < 64) {
    const int t = blockIdx.x * 64 + tid;
    if (t < T && slot_mapping[t] >= 0 && (positions[t] + 1) % pool == 0)
      list_s[atomicAdd(&count_s, 1)] = t;
  }
  __syncthreads();
  const int wave = tid / 64, lane = tid % 64;
  const int nc = (D + V) / 8, groups = 64 / nc;
  const int piece = lane % nc, grp = lane / nc;
  const bool is_k = piece * 8 < D;
  const int dd = is_k ? piece * 8 : piece * 8 - D;
  const int W = is_k ? D : V;
  const bf16* cache = is_k ? k_cache : v_cache;
  for (int i = wave; i < count_s; i += 4) {
    const int t = list_s[i];
    const int* bt = block_tables + (int64_t)token_seq[t] * max_blocks;
    const int64_t p0 = positions[t] + 1 - pool;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
#pragma unroll 4
    for (int j = grp; j < pool; j += groups) {
      const int64_t pos = p0 + j;
      const int64_t page = bt[pos / bs];
      const ushort8 u = *reinterpret_cast<const ushort8*>(
          cache + ((page * G + g) * bs + pos % bs) * W + dd);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += bf16_bits_to_float(u[e]);
    }
    for (int off = nc; off < 64; off <<= 1)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += __shfl_xor(acc[e], off, 64);
    if (grp == 0) {
      const int64_t page0 = bt[p0 / bs];
      const int e0 = (int)((p0 % bs) / pool);
      ushort8 o;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = float_to_bf16_bits(acc[e] / (float)pool);
      *reinterpret_cast<ushort8*>((is_k ? kp_cache : vp_cache) +
                                  ((page0 * G + g) * spp + e0) * W + dd) = o;
    }
  }
}

// q (fp32, LDS) . key row; 16-byte loads when rows are aligned for them
template <typename AT>
__device__ __forceinline__ float dot_row(const float* q_s, const AT* kr, int D,
                                         bool vec);
template <>
__device__ __forceinline__ float dot_row<bf16>(const float* q_s, const bf16* kr,
                                               int D, bool vec) {
  float dot = 0.f;
  if (vec) {
    for (int d = 0; d < D; d += 8) {
      const ushort8 u = *reinterpret_cast<const ushort8*>(kr + d);
#pragma unroll
      for (int e = 0; e < 8; ++e) dot += q_s[d + e] * bf16_bits_to_float(u[e]);
    }
  } else {
    for (int d = 0; d < D; ++d) dot += q_s[d] * bf16_bits_to_float(kr[d]);
  }
  return dot;
}
template <>
__device__ __forceinline__ float dot_row<float>(const float* q_s,
                                                const float* kr, int D,
                                                bool vec) {
  float dot = 0.f;
  if (vec) {
    for (int d = 0; d < D; d += 4) {
      const float4v u = *reinterpret_cast<const float4v*>(kr + d);
#pragma unroll
      for (int e = 0; e < 4; ++e) dot += q_s[d + e] * u[e];
    }
  } else {
    for (int d = 0; d < D; ++d) dot += q_s[d] * kr[d];
  }
  return dot;
}

constexpr int WP_MAX_D = 512;  // query dims held in LDS
constexpr int WP_VPT = 8;      // value dims per lane (V <= 512)

// One wave per (row, query head). The visible keys, pooled entries first and
// then the window's tokens, are visited 64 at a time: lane j scores key j,
// the wave rescales the running sums, every lane accumulates its value dims.
template <typename AT>
__global__ __launch_bounds__(64) void attn_window_pool_kernel(
    AT* __restrict__ out, int64_t ldo, const AT* __restrict__ q, int64_t ldq,
    const AT* __restrict__ k_cache, const AT* __restrict__ v_cache,
    const AT* __restrict__ kp_cache, const AT* __restrict__ vp_cache,
    const int* __restrict__ block_tables, const int* __restrict__ seq_lens,
    const int* __restrict__ cu, const int* __restrict__ token_seq, float scale,
    int window, int pool, int spp, float out_scale, int H, int G, int D, int V,
    int bs, int max_blocks) {
  __shared__ float q_s[WP_MAX_D];
  __shared__ float p_s[64];
  __shared__ const AT* vrow_s[64];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int s = token_seq[t];
  const int first_row = cu[s];
  const int rows = cu[s + 1] - first_row;
  const int pos = seq_lens[s] - rows + (t - first_row);
  const int lo = max(0, pos - window + 1);
  const int nb = pos - window + 1 > 0 ? (pos - window + 1) / pool : 0;
  const int nkeys = nb + pos - lo + 1;
  const int g = h / (H / G);
  const bool vec = D % 8 == 0;  // rows of D elements start 16 bytes apart
  const int* bt = block_tables + (int64_t)s * max_blocks;
  for (int d = lane; d < D; d += 64)
    q_s[d] = Act<AT>::ld(q + (int64_t)t * ldq + (int64_t)h * D + d);
  __syncthreads();
  float m = -INFINITY, l = 0.f;
  float acc[WP_VPT];
#pragma unroll
  for (int i = 0; i < WP_VPT; ++i) acc[i] = 0.f;
  for (int j0 = 0; j0 < nkeys; j0 += 64) {
    const int idx = j0 + lane;
    const bool valid = idx < nkeys;
    float sc = -INFINITY;
    const AT* vr = nullptr;
    if (valid) {
      const AT* kr;
      if (idx < nb) {
        const int64_t p0 = (int64_t)idx * pool;
        const int64_t e = ((int64_t)bt[p0 / bs] * G + g) * spp + (p0 % bs) / pool;
        kr = kp_cache + e * D;
        vr = vp_cache + e * V;
      } else {
        const int j = lo + idx - nb;
        const int64_t e = ((int64_t)bt[j / bs] * G + g) * bs + j % bs;
        kr = k_cache + e * D;
        vr = v_cache + e * V;
      }
      sc = dot_row<AT>(q_s, kr, D, vec) * scale;
    }
    const float m_new = fmaxf(m, wave_reduce_max(sc));
    const float p = valid ? expf(sc - m_new) : 0.f;
    const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
    l = l * corr + wave_reduce_sum(p);
#pragma unroll
    for (int i = 0; i < WP_VPT; ++i) acc[i] *= corr;
    m = m_new;
    __syncthreads();  // previous tile's readers are done
    p_s[lane] = p;
    vrow_s[lane] = vr;
    __syncthreads();
    const int cnt = min(64, nkeys - j0);
    for (int jj = 0; jj < cnt; ++jj) {
      const float pj = p_s[jj];
      const AT* vrow = vrow_s[jj];
#pragma unroll
      for (int i = 0; i < WP_VPT; ++i) {
        const int d = lane + 64 * i;
        if (d < V) acc[i] += pj * Act<AT>::ld(vrow + d);
      }
    }
  }
  const float inv = l > 0.f ? out_scale / l : 0.f;
  AT* orow = out + (int64_t)t * ldo + (int64_t)h * V;
#pragma unroll
  for (int i = 0; i < WP_VPT; ++i) {
    const int d = lane + 64 * i;
    if (d < V) Act<AT>::st(orow + d, acc[i] * inv);
  }
}

}  // namespace arks

using namespace arks;

extern "C" void arks_seq_kv_write_pooled(
    const void* k, const void* v, int64_t ldk, int64_t ldv, void* k_cache,
    void* v_cache, void* kp_cache, void* vp_cache, const void* slot_mapping,
    const void* positions, const void* block_tables, const void* token_seq,
    int T, int max_blocks, int G, int D, int V, int bs, int pool, int spp,
    int act_f32, hipStream_t stream) {
  if (T == 0) return;
  const int nc = (D + V) / 8;
  if (!act_f32 && D % 8 == 0 && V % 8 == 0 && nc <= 64 && 64 % nc == 0) {
    if (ldk % 8 == 0 && ldv % 8 == 0 &&
        (((uintptr_t)k | (uintptr_t)v) & 15) == 0)
      hipLaunchKernelGGL(kv_write_vec_kernel, dim3(T), dim3(256), 0, stream,
                         (const bf16*)k, (const bf16*)v, ldk, ldv,
                         (bf16*)k_cache, (bf16*)v_cache,
                         (const int64_t*)slot_mapping, G, D, V, bs);
    else
      hipLaunchKernelGGL((kv_write_kernel<bf16>), dim3(T), dim3(256), 0, stream,
                         (const bf16*)k, (const bf16*)v, ldk, ldv,
                         (bf16*)k_cache, (bf16*)v_cache,
                         (const int64_t*)slot_mapping, G, D, V, bs);
    hipLaunchKernelGGL(kv_pool_vec_kernel, dim3((T + 63) / 64, G), dim3(256), 0,
                       stream, (const bf16*)k_cache, (const bf16*)v_cache,
                       (bf16*)kp_cache, (bf16*)vp_cache,
                       (const int64_t*)slot_mapping, (const int64_t*)positions,
                       (const int*)block_tables, (const int*)token_seq, T,
                       max_blocks, G, D, V, bs, pool, spp);
    return;
  }
  SEQ_DISPATCH_ACT(act_f32, {
    hipLaunchKernelGGL((kv_write_kernel<AT>), dim3(T), dim3(256), 0, stream,
                       (const AT*)k, (const AT*)v, ldk, ldv, (AT*)k_cache,
                       (AT*)v_cache, (const int64_t*)slot_mapping, G, D, V, bs);
    hipLaunchKernelGGL((kv_pool_kernel<AT>), dim3((T + 63) / 64, G), dim3(256),
                       0, stream, (const AT*)k_cache, (const AT*)v_cache,
                       (AT*)kp_cache, (AT*)vp_cache,
                       (const int64_t*)slot_mapping, (const int64_t*)positions,
                       (const int*)block_tables, (const int*)token_seq, T,
                       max_blocks, G, D, V, bs, pool, spp);
  });
}

extern "C" int arks_seq_attn_window_pool(
    void* out, int64_t ldo, const void* q, int64_t ldq, const void* k_cache,
    const void* v_cache, const void* kp_cache, const void* vp_cache,
    const void* block_tables, const void* seq_lens, const void* cu,
    const void* token_seq, float scale, int window, int pool, int spp,
    float out_scale, int T, int H, int G, int D, int V, int bs, int max_blocks,
    int act_f32, hipStream_t stream) {
  if (D > WP_MAX_D || V > 64 * WP_VPT) return 1;
  if (T == 0) return 0;
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (attn_window_pool_kernel<AT>), dim3(T, H), dim3(64), 0, stream, (AT*)out,
      ldo, (const AT*)q, ldq, (const AT*)k_cache, (const AT*)v_cache,
      (const AT*)kp_cache, (const AT*)vp_cache, (const int*)block_tables,
      (const int*)seq_lens, (const int*)cu, (const int*)token_seq, scale,
      window, pool, spp, out_scale, H, G, D, V, bs, max_blocks));
  return 0;
}
