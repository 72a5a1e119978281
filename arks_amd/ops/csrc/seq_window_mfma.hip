// Sliding-window attention with pooled blocks on the matrix cores (bf16
// rows and pages of 16 tokens, gfx950): the prefill kernel of
// WindowPoolAttention (arks_amd/models/mixers.py); seq_window.hip holds the
// general kernel and the definition of the pooled caches.
//
// Tiling as in attn_extend.hip: one workgroup = 4 waves = a 64-row q tile of
// one (sequence, query head); keys pass through LDS 32 at a time (K rows
// XOR-swizzled, V as a transposed-read image) and both products run on
// v_mfma_f32_16x16x32_bf16 with an online softmax in fp32. What differs:
//   * a q tile first walks the pooled entries any of its rows may see
//     (gathered one by one from the pooled caches), then the token pages
//     from the first key its oldest row's window holds up to its last row;
//   * masks per (row, key): token j for the row at position i iff
//     i - window < j <= i; pooled block b iff (b + 1) * pool <= i - window + 1;
//   * q/k size and value size are separate template parameters, q and out
//     are row-strided views, the output is multiplied by out_scale;
//   * no host work list: workgroup y finds its (sequence, q0) by walking
//     cu_seqlens, so the launch depends on tensor shapes only;
//   * DEC (steps of single rows): a workgroup is one (row, key/value head)
//     and the tile's rows are the query heads that share it, so keys and
//     values are read once for the whole group; waves without a query head
//     only help to stage the tiles.
#include "seq_common.h"

#include <cfloat>

namespace arks {

typedef __attribute__((ext_vector_type(8))) __bf16 wp_bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 wp_bf16x4;
typedef __attribute__((ext_vector_type(4))) float wp_f32x4;

constexpr int WPM_QTILE = 64;
constexpr int WPM_KTILE = 32;
constexpr int WPM_PAGE = 16;
constexpr int WPM_PPAD = 40;

template <int D, int V, bool DEC>
__global__ __launch_bounds__(256) void attn_window_pool_mfma_kernel(
    bf16* __restrict__ out, int64_t ldo, const bf16* __restrict__ q,
    int64_t ldq, const bf16* __restrict__ k_cache,
    const bf16* __restrict__ v_cache, const bf16* __restrict__ kp_cache,
    const bf16* __restrict__ vp_cache, const int* __restrict__ block_tables,
    const int* __restrict__ kv_lens, const int* __restrict__ cu,
    const int* __restrict__ token_seq, int num_seqs, float scale, int window,
    int pool, int spp, float out_scale, int G, int H, int max_blocks) {
  constexpr int STEPS = D / 32;
  constexpr int CHUNKS = V / 16;
  constexpr int SWZ = ((D & (D - 1)) == 0 && D >= 64) ? 1 : 0;

  // which q tile is this workgroup's
  int seq_idx = -1, q0 = 0;
  if (DEC) {
    seq_idx = token_seq[blockIdx.y];
    q0 = blockIdx.y - cu[seq_idx];
  } else {
    int left = blockIdx.y;
    for (int s = 0; s < num_seqs; ++s) {
      const int n = (cu[s + 1] - cu[s] + WPM_QTILE - 1) / WPM_QTILE;
      if (left < n) {
        seq_idx = s;
        q0 = left * WPM_QTILE;
        break;
      }
      left -= n;
    }
  }
  if (seq_idx < 0) return;
  const int GQ = H / G;
  const int kvh = DEC ? blockIdx.x : blockIdx.x / GQ;
  const int q_start = cu[seq_idx];
  const int q_len = cu[seq_idx + 1] - q_start;
  const int kv_len = kv_lens[seq_idx];
  const int kv_off = kv_len - q_len;
  const int* __restrict__ bt = block_tables + (int64_t)seq_idx * max_blocks;

  const int tid = threadIdx.x;
  const int wave = tid / WAVE_SIZE, lane = tid % WAVE_SIZE;
  const int lq = lane % 16, la = lane / 16;

  __shared__ __attribute__((aligned(16))) bf16 k_lds[WPM_KTILE][D];
  __shared__ __attribute__((aligned(16))) bf16 vt_img[V / 16][8][96];
  __shared__ __attribute__((aligned(16))) bf16 p_lds[4][16][WPM_PPAD];

  // this lane's score column: a row of the sequence, or (DEC) a query head
  // of the group, all at the one row's position
  const int my_qrow = DEC ? q0 : q0 + wave * 16 + lq;
  const bool qrow_valid = DEC ? wave * 16 + lq < GQ : my_qrow < q_len;
  const int h = DEC ? kvh * GQ + (qrow_valid ? wave * 16 + lq : 0) : blockIdx.x;
  const bool wave_active = !DEC || wave * 16 < GQ;
  const int my_pos = kv_off + my_qrow;
  // pooled blocks this lane's row sees
  const int my_nb = my_pos - window + 1 > 0 ? (my_pos - window + 1) / pool : 0;
  wp_bf16x8 qfrag[STEPS];
  {
    const int64_t qbase =
        (int64_t)(q_start + (qrow_valid ? my_qrow : 0)) * ldq + (int64_t)h * D;
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
      ushort8 u = *reinterpret_cast<const ushort8*>(q + qbase + st * 32 + 8 * la);
      qfrag[st] = *reinterpret_cast<wp_bf16x8*>(&u);
    }
  }

  float m_run = -FLT_MAX, l_run = 0.f;
  wp_f32x4 oacc[CHUNKS];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) oacc[c] = {0.f, 0.f, 0.f, 0.f};

  const int last_pos = DEC ? my_pos : kv_off + min(q0 + WPM_QTILE, q_len) - 1;
  const int nb_max = last_pos - window + 1 > 0 ? (last_pos - window + 1) / pool : 0;
  const int pool_tiles = (nb_max + WPM_KTILE - 1) / WPM_KTILE;
  const int kmax = last_pos + 1;
  const int tok_j0 = max(0, kv_off + q0 - window + 1) / WPM_KTILE;
  static_assert(WPM_QTILE == 64, "four waves of 16 rows");
  const int tok_tiles = (kmax + WPM_KTILE - 1) / WPM_KTILE;
  const int n_iter = pool_tiles + (tok_tiles - tok_j0);

  for (int it = 0; it < n_iter; ++it) {
    const bool pooled = it < pool_tiles;
    const int key_base = pooled ? it * WPM_KTILE : (tok_j0 + it - pool_tiles) * WPM_KTILE;
    const int key_end = pooled ? nb_max : kmax;
    for (int i = tid; i < WPM_KTILE * (D / 8); i += 256) {
      const int key = i / (D / 8);
      const int col8 = (i % (D / 8)) * 8;
      const int kg = key_base + key;
      ushort8 kv{};
      if (kg < key_end) {
        int64_t src;
        if (pooled) {
          const int64_t p0 = (int64_t)kg * pool;
          src = (((int64_t)bt[p0 / WPM_PAGE] * G + kvh) * spp +
                 (p0 % WPM_PAGE) / pool) * D;
          kv = *reinterpret_cast<const ushort8*>(kp_cache + src + col8);
        } else {
          src = (((int64_t)bt[kg / WPM_PAGE] * G + kvh) * WPM_PAGE +
                 kg % WPM_PAGE) * D;
          kv = *reinterpret_cast<const ushort8*>(k_cache + src + col8);
        }
      }
      const int swz = (col8 * 2) ^ (SWZ * ((key & 7) << 4));
      *reinterpret_cast<ushort8*>(reinterpret_cast<char*>(&k_lds[key][0]) + swz) = kv;
    }
    for (int i = tid; i < WPM_KTILE * (V / 8); i += 256) {
      const int key = i / (V / 8);
      const int col8 = (i % (V / 8)) * 8;
      const int kg = key_base + key;
      ushort8 vv{};
      if (kg < key_end) {
        int64_t src;
        if (pooled) {
          const int64_t p0 = (int64_t)kg * pool;
          src = (((int64_t)bt[p0 / WPM_PAGE] * G + kvh) * spp +
                 (p0 % WPM_PAGE) / pool) * V;
          vv = *reinterpret_cast<const ushort8*>(vp_cache + src + col8);
        } else {
          src = (((int64_t)bt[kg / WPM_PAGE] * G + kvh) * WPM_PAGE +
                 kg % WPM_PAGE) * V;
          vv = *reinterpret_cast<const ushort8*>(v_cache + src + col8);
        }
      }
      *reinterpret_cast<ushort8*>(
          &vt_img[col8 >> 4][key >> 2][(key & 3) * 16 + (col8 & 15)]) = vv;
    }
    __syncthreads();

    if (wave_active) {
    wp_f32x4 sc[2];
    sc[0] = {0.f, 0.f, 0.f, 0.f};
    sc[1] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      const int key = sub * 16 + lq;
#pragma unroll
      for (int st = 0; st < STEPS; ++st) {
        const int col_byte = (st * 32 + 8 * la) * 2;
        const int swz = col_byte ^ (SWZ * ((key & 7) << 4));
        ushort8 u = *reinterpret_cast<const ushort8*>(
            reinterpret_cast<const char*>(&k_lds[key][0]) + swz);
        sc[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            *reinterpret_cast<wp_bf16x8*>(&u), qfrag[st], sc[sub], 0, 0, 0);
      }
    }

    float p[8];
    bool msk[8];
    float tile_max = -FLT_MAX;
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int kg = key_base + sub * 16 + 4 * la + r;
        const int i = sub * 4 + r;
        msk[i] = qrow_valid &&
                 (pooled ? kg < my_nb : (kg <= my_pos && kg > my_pos - window));
        p[i] = msk[i] ? sc[sub][r] * scale : -FLT_MAX;
        tile_max = fmaxf(tile_max, p[i]);
      }
    }
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, WAVE_SIZE));
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, WAVE_SIZE));
    const float m_new = fmaxf(m_run, tile_max);
    float alpha = 1.f, psum = 0.f;
    if (m_new > -FLT_MAX) {
      alpha = __expf(m_run - m_new);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        p[i] = msk[i] ? __expf(p[i] - m_new) : 0.f;
        psum += p[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) p[i] = 0.f;
    }
    psum += __shfl_xor(psum, 16, WAVE_SIZE);
    psum += __shfl_xor(psum, 32, WAVE_SIZE);
    l_run = l_run * alpha + psum;
    m_run = m_new;

    float row_alpha[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) row_alpha[r] = __shfl(alpha, 4 * la + r, WAVE_SIZE);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
      for (int r = 0; r < 4; ++r) oacc[c][r] *= row_alpha[r];

#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      ushort4v pk;
#pragma unroll
      for (int r = 0; r < 4; ++r) pk[r] = float_to_bf16_bits(p[sub * 4 + r]);
      *reinterpret_cast<ushort4v*>(&p_lds[wave][lq][sub * 16 + 4 * la]) = pk;
    }
    }
    __syncthreads();

    if (wave_active) {
    ushort8 pa = *reinterpret_cast<const ushort8*>(&p_lds[wave][lq][8 * la]);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      wp_bf16x4 v1 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
          (__attribute__((address_space(3))) wp_bf16x4*)(
              reinterpret_cast<char*>(&vt_img[c][2 * la][0]) + lq * 8));
      wp_bf16x4 v2 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
          (__attribute__((address_space(3))) wp_bf16x4*)(
              reinterpret_cast<char*>(&vt_img[c][2 * la + 1][0]) + lq * 8));
      wp_bf16x8 vb;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        vb[e] = v1[e];
        vb[e + 4] = v2[e];
      }
      oacc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
          *reinterpret_cast<wp_bf16x8*>(&pa), vb, oacc[c], 0, 0, 0);
    }
    }
    __syncthreads();
  }

  float row_inv[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float lr = __shfl(l_run, 4 * la + r, WAVE_SIZE);
    row_inv[r] = lr > 0.f ? out_scale / lr : 0.f;
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int sub = wave * 16 + 4 * la + r;  // row of the tile
    if (DEC ? sub >= GQ : q0 + sub >= q_len) continue;
    const int64_t obase =
        DEC ? (int64_t)(q_start + q0) * ldo + (int64_t)(kvh * GQ + sub) * V
            : (int64_t)(q_start + q0 + sub) * ldo + (int64_t)blockIdx.x * V;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c)
      out[obase + c * 16 + lq] = float_to_bf16_bits(oacc[c][r] * row_inv[r]);
  }
}

// Single rows, groups of up to 16 query heads: one workgroup per (row,
// key/value head) whose four waves each take every fourth 32-key tile of
// the visible keys (pooled entries first) with no barrier between tiles —
// K goes from the pages straight into the MFMA A operand, V through a
// per-wave transposed-read image, P through a per-wave tile — and merge
// their (max, sum, output) partials through LDS at the end. The heads of
// the group are the columns of the score tile, so keys and values are read
// once for all of them.
template <int D, int V>
__global__ __launch_bounds__(256) void attn_window_pool_dec_kernel(
    bf16* __restrict__ out, int64_t ldo, const bf16* __restrict__ q,
    int64_t ldq, const bf16* __restrict__ k_cache,
    const bf16* __restrict__ v_cache, const bf16* __restrict__ kp_cache,
    const bf16* __restrict__ vp_cache, const int* __restrict__ block_tables,
    const int* __restrict__ kv_lens, const int* __restrict__ cu,
    const int* __restrict__ token_seq, float scale, int window, int pool,
    int spp, float out_scale, int G, int H, int max_blocks) {
  constexpr int STEPS = D / 32;
  constexpr int CHUNKS = V / 16;
  constexpr int E = V / 16;  // value dims per thread in the merge
  const int t = blockIdx.y, kvh = blockIdx.x;
  const int GQ = H / G;
  const int seq = token_seq[t];
  const int q_start = cu[seq];
  const int pos = kv_lens[seq] - (cu[seq + 1] - q_start) + (t - q_start);
  const int* __restrict__ bt = block_tables + (int64_t)seq * max_blocks;
  const int tid = threadIdx.x;
  const int wave = tid / WAVE_SIZE, lane = tid % WAVE_SIZE;
  const int lq = lane % 16, la = lane / 16;

  constexpr int VT_BYTES = (V / 16) * 8 * 96 * 2;
  constexpr int P_BYTES = 16 * WPM_PPAD * 2;
  constexpr int MERGE_BYTES = 16 * (V + 2) * 4;
  constexpr int WAVE_BYTES0 =
      VT_BYTES + P_BYTES > MERGE_BYTES ? VT_BYTES + P_BYTES : MERGE_BYTES;
  constexpr int WAVE_BYTES = (WAVE_BYTES0 + 15) & ~15;
  __shared__ __attribute__((aligned(16))) char smem[4][WAVE_BYTES];
  bf16* vt_lds = reinterpret_cast<bf16*>(smem[wave]);
  bf16* p_lds = reinterpret_cast<bf16*>(smem[wave] + VT_BYTES);
  float* merge_lds = reinterpret_cast<float*>(smem[wave]);

  wp_bf16x8 qfrag[STEPS];
  {
    const bool valid = lq < GQ;
    const bf16* qp = q + (int64_t)t * ldq + (int64_t)(kvh * GQ + (valid ? lq : 0)) * D;
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
      ushort8 u{};
      if (valid) u = *reinterpret_cast<const ushort8*>(qp + st * 32 + 8 * la);
      qfrag[st] = *reinterpret_cast<wp_bf16x8*>(&u);
    }
  }
  float m_run = -FLT_MAX, l_run = 0.f;
  wp_f32x4 oacc[CHUNKS];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) oacc[c] = {0.f, 0.f, 0.f, 0.f};

  const int nb = pos - window + 1 > 0 ? (pos - window + 1) / pool : 0;
  const int lo = max(0, pos - window + 1);
  const int pool_tiles = (nb + WPM_KTILE - 1) / WPM_KTILE;
  const int tok_j0 = lo / WPM_KTILE;
  const int n_iter = pool_tiles + (pos + 1 + WPM_KTILE - 1) / WPM_KTILE - tok_j0;
  // first element of key kg's row in its cache, in units of rows
  auto row_of = [&](bool pooled, int kg) -> int64_t {
    if (pooled) {
      const int64_t p0 = (int64_t)kg * pool;
      return ((int64_t)bt[p0 / WPM_PAGE] * G + kvh) * spp + (p0 % WPM_PAGE) / pool;
    }
    return ((int64_t)bt[kg / WPM_PAGE] * G + kvh) * WPM_PAGE + kg % WPM_PAGE;
  };
  constexpr int NV = WPM_KTILE * V / 8 / WAVE_SIZE;

  // tile `it` of this wave's keys into registers: K as the MFMA A operand
  // (key lq of each 16-key half, 8 dims per lane and step), V as 16-byte
  // pieces for the transposed-read image; keys past the end read as zeros
  auto load_tile = [&](int it, ushort8 (&kr)[2][STEPS], ushort8 (&vr)[NV]) {
    const bool pooled = it < pool_tiles;
    const int key_base =
        pooled ? it * WPM_KTILE : (tok_j0 + it - pool_tiles) * WPM_KTILE;
    const int key_end = pooled ? nb : pos + 1;
    const bf16* kc = pooled ? kp_cache : k_cache;
    const bf16* vc = pooled ? vp_cache : v_cache;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int i = lane + WAVE_SIZE * j;
      const int key = i / (V / 8);
      const int col8 = (i % (V / 8)) * 8;
      ushort8 v{};
      if (key_base + key < key_end)
        v = *reinterpret_cast<const ushort8*>(
            vc + row_of(pooled, key_base + key) * V + col8);
      vr[j] = v;
    }
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      const int kg = key_base + sub * 16 + lq;
      const bool have = kg < key_end;
      const bf16* krow = kc + (have ? row_of(pooled, kg) : 0) * D + 8 * la;
#pragma unroll
      for (int st = 0; st < STEPS; ++st) {
        ushort8 u{};
        if (have) u = *reinterpret_cast<const ushort8*>(krow + st * 32);
        kr[sub][st] = u;
      }
    }
  };
  ushort8 kreg[2][STEPS], vv[NV];
  if (wave < n_iter) load_tile(wave, kreg, vv);

  for (int it = wave; it < n_iter; it += 4) {
    const bool pooled = it < pool_tiles;
    const int key_base =
        pooled ? it * WPM_KTILE : (tok_j0 + it - pool_tiles) * WPM_KTILE;
    // the next tile's loads fly while this one computes
    ushort8 knext[2][STEPS], vnext[NV];
    if (it + 4 < n_iter) load_tile(it + 4, knext, vnext);
    wp_f32x4 sc[2];
    sc[0] = {0.f, 0.f, 0.f, 0.f};
    sc[1] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int sub = 0; sub < 2; ++sub)
#pragma unroll
      for (int st = 0; st < STEPS; ++st)
        sc[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            *reinterpret_cast<wp_bf16x8*>(&kreg[sub][st]), qfrag[st], sc[sub],
            0, 0, 0);
    float p[8];
    float tile_max = -FLT_MAX;
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int kg = key_base + sub * 16 + 4 * la + r;
        const int i = sub * 4 + r;
        const bool vis = pooled ? kg < nb : (kg <= pos && kg > pos - window);
        p[i] = vis ? sc[sub][r] * scale : -FLT_MAX;
        tile_max = fmaxf(tile_max, p[i]);
      }
    }
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, WAVE_SIZE));
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, WAVE_SIZE));
    const float m_new = fmaxf(m_run, tile_max);
    float alpha = 1.f, psum = 0.f;
    if (m_new > -FLT_MAX) {
      alpha = __expf(m_run - m_new);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        p[i] = (p[i] > -FLT_MAX) ? __expf(p[i] - m_new) : 0.f;
        psum += p[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) p[i] = 0.f;
    }
    psum += __shfl_xor(psum, 16, WAVE_SIZE);
    psum += __shfl_xor(psum, 32, WAVE_SIZE);
    l_run = l_run * alpha + psum;
    m_run = m_new;
    float row_alpha[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) row_alpha[r] = __shfl(alpha, 4 * la + r, WAVE_SIZE);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
      for (int r = 0; r < 4; ++r) oacc[c][r] *= row_alpha[r];
    // V into the transposed-read image; LDS runs in order within a wave, so
    // these stores land after the previous tile's reads
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int i = lane + WAVE_SIZE * j;
      const int key = i / (V / 8);
      const int col8 = (i % (V / 8)) * 8;
      *reinterpret_cast<ushort8*>(
          &vt_lds[((col8 >> 4) * 8 + (key >> 2)) * 96 + (key & 3) * 16 +
                  (col8 & 15)]) = vv[j];
    }
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      ushort4v pk;
#pragma unroll
      for (int r = 0; r < 4; ++r) pk[r] = float_to_bf16_bits(p[sub * 4 + r]);
      *reinterpret_cast<ushort4v*>(&p_lds[lq * WPM_PPAD + sub * 16 + 4 * la]) = pk;
    }
    // producer -> consumer between lanes of this wave: the LDS counter only
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    ushort8 pa = *reinterpret_cast<const ushort8*>(&p_lds[lq * WPM_PPAD + 8 * la]);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      wp_bf16x4 v1 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
          (__attribute__((address_space(3))) wp_bf16x4*)(
              reinterpret_cast<char*>(&vt_lds[(c * 8 + 2 * la) * 96]) + lq * 8));
      wp_bf16x4 v2 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
          (__attribute__((address_space(3))) wp_bf16x4*)(
              reinterpret_cast<char*>(&vt_lds[(c * 8 + 2 * la + 1) * 96]) + lq * 8));
      wp_bf16x8 vb;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        vb[e] = v1[e];
        vb[e + 4] = v2[e];
      }
      oacc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
          *reinterpret_cast<wp_bf16x8*>(&pa), vb, oacc[c], 0, 0, 0);
    }
    if (it + 4 < n_iter) {
#pragma unroll
      for (int sub = 0; sub < 2; ++sub)
#pragma unroll
        for (int st = 0; st < STEPS; ++st) kreg[sub][st] = knext[sub][st];
#pragma unroll
      for (int j = 0; j < NV; ++j) vv[j] = vnext[j];
    }
  }

  __syncthreads();  // every wave is done with its tiles before the union flips
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      merge_lds[(4 * la + r) * (V + 2) + c * 16 + lq] = oacc[c][r];
  if (la == 0) {
    merge_lds[lq * (V + 2) + V] = m_run;
    merge_lds[lq * (V + 2) + V + 1] = l_run;
  }
  __syncthreads();
  // 256 threads = 16 heads x 16 slices of the value dims
  const int g = tid / 16, lane16 = tid % 16;
  if (g >= GQ) return;
  float mf = -FLT_MAX, lf = 0.f, af[E];
#pragma unroll
  for (int e = 0; e < E; ++e) af[e] = 0.f;
  for (int w = 0; w < 4; ++w) {
    const float* wl = reinterpret_cast<const float*>(smem[w]);
    const float mw = wl[g * (V + 2) + V];
    const float lw = wl[g * (V + 2) + V + 1];
    const float mn = fmaxf(mf, mw);
    const float a1 = __expf(mf - mn), a2 = __expf(mw - mn);
    lf = lf * a1 + lw * a2;
#pragma unroll
    for (int e = 0; e < E; ++e)
      af[e] = af[e] * a1 + wl[g * (V + 2) + lane16 * E + e] * a2;
    mf = mn;
  }
  const float inv = lf > 0.f ? out_scale / lf : 0.f;
  bf16* op = out + (int64_t)t * ldo + (int64_t)(kvh * GQ + g) * V + lane16 * E;
#pragma unroll
  for (int e = 0; e < E; ++e) op[e] = float_to_bf16_bits(af[e] * inv);
}

}  // namespace arks

using namespace arks;

// Returns 1 when no kernel is built for these sizes (the caller then runs
// the general kernel).
extern "C" int arks_seq_attn_window_pool_mfma(
    void* out, int64_t ldo, const void* q, int64_t ldq, const void* k_cache,
    const void* v_cache, const void* kp_cache, const void* vp_cache,
    const void* block_tables, const void* seq_lens, const void* cu,
    const void* token_seq, float scale, int window, int pool, int spp,
    float out_scale, int T, int H, int G, int D, int V, int bs, int max_blocks,
    int num_seqs, int single_rows, hipStream_t stream) {
  if (bs != WPM_PAGE || ldq % 8 || H % G || ((uintptr_t)q & 15)) return 1;
  if (single_rows && H / G > WPM_QTILE) return 1;
  if (T == 0) return 0;
  // prompts: every sequence adds at most one partly filled tile
  dim3 grid(H, (T + WPM_QTILE - 1) / WPM_QTILE + num_seqs), block(256);
  if (single_rows) grid = dim3(G, T);
#define WPM_ARGS                                                              \
  grid, block, 0, stream, (bf16*)out, ldo, (const bf16*)q, ldq,               \
      (const bf16*)k_cache, (const bf16*)v_cache, (const bf16*)kp_cache,      \
      (const bf16*)vp_cache, (const int*)block_tables, (const int*)seq_lens,  \
      (const int*)cu, (const int*)token_seq, num_seqs, scale, window, pool,   \
      spp, out_scale, G, H, max_blocks
#define WPM(DD, VV)                                                           \
  if (D == DD && V == VV) {                                                   \
    if (single_rows && H / G <= 16)                                           \
      hipLaunchKernelGGL((attn_window_pool_dec_kernel<DD, VV>), grid, block,  \
                         0, stream, (bf16*)out, ldo, (const bf16*)q, ldq,      \
                         (const bf16*)k_cache, (const bf16*)v_cache,           \
                         (const bf16*)kp_cache, (const bf16*)vp_cache,         \
                         (const int*)block_tables, (const int*)seq_lens,       \
                         (const int*)cu, (const int*)token_seq, scale, window, \
                         pool, spp, out_scale, G, H, max_blocks);              \
    else if (single_rows)                                                     \
      hipLaunchKernelGGL((attn_window_pool_mfma_kernel<DD, VV, true>),        \
                         WPM_ARGS);                                           \
    else                                                                      \
      hipLaunchKernelGGL((attn_window_pool_mfma_kernel<DD, VV, false>),       \
                         WPM_ARGS);                                           \
    return 0;                                                                 \
  }
  WPM(64, 64)
  WPM(128, 128)
  WPM(128, 64)
  WPM(64, 128)
  WPM(32, 32)
  WPM(96, 96)
#undef WPM
#undef WPM_ARGS
  return 1;
}
