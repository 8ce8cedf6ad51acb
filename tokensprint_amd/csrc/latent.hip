// Attention over a shared low-rank latent kept in pages: every cached token is one row
// [c (kv_rank) | k_r (rot_dim)] that all heads read, as key (all of it) and as value (c).
// Queries arrive already carried into that space, q' = [U_k^T q_n | rot(q_r)], and the
// result leaves as sum_t p_t c_t per head, for the value up-projection behind it.
//
// Kernels: the preparation of a step's rows (norms of the two latents, rotation of the
// shared key part, the write into the pages), the rotation of the queries' rotated part in
// place, and attention.  (Carrying queries into the latent's space and results out of it
// are plain products over weights folded at load.)
// Scores, softmax, rotation angles, norms: float32.  The rotation pairs dimension 2i with
// 2i+1 and turns them by position * freq[i]; cosine and sine are computed here, at the
// position, so there is no table and no longest position.
#include "common.h"

typedef __attribute__((ext_vector_type(4))) float f32x4_l;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_l;
__device__ __forceinline__ f32x4_l load4_l(const float* p) { return *(const f32x4_l*)p; }
__device__ __forceinline__ f32x4_l load4_l(const bf16_t* p) {
  const bf16x4_l v = *(const bf16x4_l*)p;
  return f32x4_l{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}

__device__ __forceinline__ void rotate_pair(float u, float v, int pos, float freq, float* ou,
                                            float* ov) {
  float sn, cs;
  sincosf((float)pos * freq, &sn, &cs);
  *ou = u * cs - v * sn;
  *ov = v * cs + u * sn;
}

// ---------------------------------------------------------------- preparation
// proj row: [q latent (q_rank) | kv latent (kv_rank) | shared key part (rot_dim)], float32.
// cq = q latent / rms * q_norm -> out (the up-projection's input);
// c = kv latent / rms * kv_norm and the rotated key part -> the token's row in the pages.
template <typename TO, typename TC>
__global__ __launch_bounds__(256) void latent_prepare_kernel(
    const float* __restrict__ proj, const float* __restrict__ q_norm,
    const float* __restrict__ kv_norm, const float* __restrict__ freqs, TO* __restrict__ cq,
    TC* __restrict__ pages, const int* __restrict__ positions,
    const int* __restrict__ entry_of_token, const int* __restrict__ table, int table_width,
    int page_size, int q_rank, int kv_rank, int rot_dim, int rot_dims, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const int ld = q_rank + kv_rank + rot_dim, dl = kv_rank + rot_dim;
  const float* row = proj + (int64_t)t * ld;
  float sq = 0.f, sc = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) sq += row[i] * row[i];
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) sc += row[q_rank + i] * row[q_rank + i];
  const float rq = 1.0f / sqrtf(block_sum(sq, scratch) / (float)q_rank + eps);
  const float rc = 1.0f / sqrtf(block_sum(sc, scratch) / (float)kv_rank + eps);
  TO* o = cq + (int64_t)t * q_rank;
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) o[i] = from_f32<TO>(row[i] * rq * q_norm[i]);
  const int pos = positions[t];
  const int page = table[(int64_t)entry_of_token[t] * table_width + pos / page_size];
  if (page < 0) return;     // an idle lane of a fixed-size batch: nothing to keep
  TC* dst = pages + ((int64_t)page * page_size + pos % page_size) * dl;
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x)
    dst[i] = from_f32<TC>(row[q_rank + i] * rc * kv_norm[i]);
  const float* kr = row + q_rank + kv_rank;
  for (int i = threadIdx.x; i < rot_dim / 2 + rot_dim % 2; i += blockDim.x) {
    if (2 * i + 1 < rot_dims) {
      float u, v;
      rotate_pair(kr[2 * i], kr[2 * i + 1], pos, freqs[i], &u, &v);
      dst[kv_rank + 2 * i] = from_f32<TC>(u);
      dst[kv_rank + 2 * i + 1] = from_f32<TC>(v);
    } else {
      dst[kv_rank + 2 * i] = from_f32<TC>(kr[2 * i]);
      if (2 * i + 1 < rot_dim) dst[kv_rank + 2 * i + 1] = from_f32<TC>(kr[2 * i + 1]);
    }
  }
}

extern "C" int ts_latent_prepare(const float* proj, const float* q_norm, const float* kv_norm,
                                 const float* freqs, void* cq, int out_type, void* pages,
                                 int cache_type, const int* positions,
                                 const int* entry_of_token, const int* table, int table_width,
                                 int page_size, int num_tokens, int q_rank, int kv_rank,
                                 int rot_dim, int rot_dims, float eps, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (q_rank <= 0 || kv_rank <= 0 || rot_dim < 0 || rot_dims % 2 || rot_dims > rot_dim ||
      page_size <= 0 || table_width <= 0)
    TS_FAIL("latent_prepare: bad sizes q_rank=%d kv_rank=%d rot_dim=%d rot_dims=%d", q_rank,
            kv_rank, rot_dim, rot_dims);
  TS_DISPATCH_TYPE(out_type, TO, TS_DISPATCH_TYPE(cache_type, TC,
      hipLaunchKernelGGL((latent_prepare_kernel<TO, TC>), dim3(num_tokens), dim3(256), 0, stream,
                         proj, q_norm, kv_norm, freqs, (TO*)cq, (TC*)pages, positions,
                         entry_of_token, table, table_width, page_size, q_rank, kv_rank, rot_dim,
                         rot_dims, eps)));
  TS_CHECK_LAUNCH("latent_prepare");
  return 0;
}

// ---------------------------------------------------------------- rotation in place
// x [T, heads, width]: the pairs (offset + 2i, offset + 2i + 1), i < dims / 2, of every
// head's vector are turned by positions[t] * freqs[i].
template <typename T>
__global__ __launch_bounds__(256) void rotate_interleaved_kernel(
    T* __restrict__ x, const int* __restrict__ positions, const float* __restrict__ freqs,
    int64_t total, int heads, int width, int offset, int half) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int i = (int)(idx % half);
  const int64_t th = idx / half;                      // token * heads + head
  T* v = x + th * width + offset + 2 * i;
  float a, b;
  rotate_pair(to_f32(v[0]), to_f32(v[1]), positions[th / heads], freqs[i], &a, &b);
  v[0] = from_f32<T>(a);
  v[1] = from_f32<T>(b);
}

extern "C" int ts_rotate_interleaved(void* x, int type, const int* positions, const float* freqs,
                                     int num_tokens, int heads, int width, int offset, int dims,
                                     hipStream_t stream) {
  if (num_tokens <= 0 || dims == 0) return 0;
  if (heads <= 0 || dims % 2 || offset < 0 || offset + dims > width)
    TS_FAIL("rotate_interleaved: bad sizes heads=%d width=%d offset=%d dims=%d", heads, width,
            offset, dims);
  const int64_t total = (int64_t)num_tokens * heads * (dims / 2);
  TS_DISPATCH_TYPE(type, T,
                   hipLaunchKernelGGL(rotate_interleaved_kernel<T>,
                                      dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                                      (T*)x, positions, freqs, total, heads, width, offset,
                                      dims / 2));
  TS_CHECK_LAUNCH("rotate_interleaved");
  return 0;
}

// ---------------------------------------------------------------- attention
// One wavefront per (token, head), four heads of a token to a workgroup (they read the same
// rows).  Keys are cut into tiles of 64 starting at the first visible key, so the partition
// and with it the rounding depends only on the token's position and the window.  In a
// tile, lane j scores key j (a dot product over the whole row); then the lanes turn to the
// columns of c and add the tile's weighted rows, key by key in order.
constexpr int kMaxLatent = 2048;              // kv_rank + rot_dim
constexpr int kLatentWaves = 4;
constexpr int kMaxRankPerLane = 16;           // kv_rank <= 1024

template <typename TC, typename TO>
__global__ __launch_bounds__(kLatentWaves* kWave) void latent_attention_kernel(
    const float* __restrict__ qa, const TC* __restrict__ pages, TO* __restrict__ out,
    const int* __restrict__ positions, const int* __restrict__ entry_of_token,
    const int* __restrict__ table, int table_width, int page_size, int heads, int kv_rank,
    int rot_dim, int window, float scale) {
  extern __shared__ float lds[];      // per wave: q [dl], p [64], row numbers [64]
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int dl = kv_rank + rot_dim;
  const int per_wave = dl + 2 * kWave;
  float* q_s = lds + (size_t)wave * per_wave;
  float* p_s = q_s + dl;
  int* row_s = (int*)(p_s + kWave);
  const int t = blockIdx.x;
  const int h = blockIdx.y * kLatentWaves + wave;
  if (h >= heads) return;             // waves are independent: no workgroup barrier below
  const int pos = positions[t];
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int* tab = table + (int64_t)entry_of_token[t] * table_width;
  const float* q = qa + ((int64_t)t * heads + h) * dl;
  for (int d = lane; d < dl; d += kWave) q_s[d] = q[d];
  __builtin_amdgcn_wave_barrier();
  const bool by4 = dl % 4 == 0 && ((uintptr_t)pages & 15) == 0;

  float m = -INFINITY, l = 0.f;
  float acc[kMaxRankPerLane] = {};
  for (int j0 = lo; j0 <= pos; j0 += kWave) {
    const int j = j0 + lane;
    float s = -INFINITY;
    int row = -1;               // the token's row in the pages
    if (j <= pos) {
      const int page = tab[j / page_size];
      if (page >= 0) {
        row = page * page_size + j % page_size;
        const TC* kr = pages + (int64_t)row * dl;
        float dot = 0.f;
        if (by4) {
          for (int d = 0; d < dl; d += 4) {
            const f32x4_l k4 = load4_l(kr + d);
#pragma unroll
            for (int e = 0; e < 4; ++e) dot = fmaf(q_s[d + e], k4[e], dot);
          }
        } else {
          for (int d = 0; d < dl; ++d) dot = fmaf(q_s[d], to_f32(kr[d]), dot);
        }
        s = dot * scale;
      }
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float corr = m_new == -INFINITY ? 1.f : expf(m - m_new);
    const float p = (row >= 0 && m_new != -INFINITY) ? expf(s - m_new) : 0.f;
    l = l * corr + wave_sum(p);
    m = m_new;
    p_s[lane] = p;
    row_s[lane] = row;
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int r = 0; r < kMaxRankPerLane; ++r) acc[r] *= corr;
    const int n = min(kWave, pos - j0 + 1);
    for (int jj = 0; jj < n; ++jj) {
      if (row_s[jj] < 0) continue;
      const int64_t vr = (int64_t)row_s[jj] * dl;
      const float pj = p_s[jj];
#pragma unroll
      for (int r = 0; r < kMaxRankPerLane; ++r) {
        const int d = lane + r * kWave;
        if (d < kv_rank) acc[r] = fmaf(pj, to_f32(pages[vr + d]), acc[r]);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  TO* o = out + ((int64_t)t * heads + h) * kv_rank;
  const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
  for (int r = 0; r < kMaxRankPerLane; ++r) {
    const int d = lane + r * kWave;
    if (d < kv_rank) o[d] = from_f32<TO>(acc[r] * inv);
  }
}

extern "C" int ts_latent_attention(const float* qa, const void* pages, int cache_type, void* out,
                                   int out_type, const int* positions, const int* entry_of_token,
                                   const int* table, int table_width, int page_size,
                                   int num_tokens, int heads, int kv_rank, int rot_dim,
                                   int window, float scale, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  const int dl = kv_rank + rot_dim;
  if (heads <= 0 || kv_rank <= 0 || rot_dim < 0 || page_size <= 0 || table_width <= 0)
    TS_FAIL("latent_attention: bad sizes heads=%d kv_rank=%d rot_dim=%d", heads, kv_rank, rot_dim);
  if (kv_rank > kMaxRankPerLane * kWave || dl > kMaxLatent)
    TS_FAIL("latent_attention: latent of %d + %d elements, at most %d + %d are built", kv_rank,
            rot_dim, kMaxRankPerLane * kWave, kMaxLatent - kMaxRankPerLane * kWave);
  const size_t lds = (size_t)kLatentWaves * (dl + 2 * kWave) * sizeof(float);
  const dim3 grid(num_tokens, (heads + kLatentWaves - 1) / kLatentWaves);
  TS_DISPATCH_TYPE(cache_type, TC, TS_DISPATCH_TYPE(out_type, TO,
      hipLaunchKernelGGL((latent_attention_kernel<TC, TO>), grid, dim3(kLatentWaves * kWave), lds,
                         stream, qa, (const TC*)pages, (TO*)out, positions, entry_of_token, table,
                         table_width, page_size, heads, kv_rank, rot_dim, window, scale)));
  TS_CHECK_LAUNCH("latent_attention");
  return 0;
}


// ---------------------------------------------------------------- attention on the matrix cores
// bfloat16 pages.  A tile is 16 consecutive rows of the step's (token, head) rows that
// belong to one entry: every head reads the same cached rows, so a decode step's token is
// one tile of its heads, and a prompt's tile a few tokens with all their heads.  One
// wavefront per (tile, share of the keys):
//     S^T = K Q'^T        v_mfma_f32_16x16x32_bf16, reduction over the latent row
//     O^T += C^T P^T      the same instruction, reduction over 32 keys
// Lane (r, g) = (lane % 16, lane / 16) owns query row r: its scores come out as
// S^T[key 4g + t][row r], which is, in place, its part of the second product's B operand;
// its softmax statistics are shared with lanes r + 16, r + 32, r + 48; its part of O^T is
// [columns 16 db + 4g + t][row r], so rescaling needs nothing from other lanes.
// Keys are walked in blocks of 32 at absolute multiples of 32.  Where a step has few
// tiles, a tile's keys are shared out in runs of `keys_per_split` over several wavefronts,
// whose unnormalised results and statistics a second kernel merges.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_l;

struct LatentMfmaArgs {
  const float* qa;          // [rows, dl], rows = tokens * heads
  const bf16_t* pages;      // [pages, page_size, dl]
  void* out;                // [rows, kv_rank]
  const int* tiles;         // [num_tiles, 3]: first row, rows (1..16), entry
  const int* positions;     // [tokens]
  const int* table;
  float* part_o;            // [num_tiles, splits, 16, kv_rank]
  float* part_ml;           // [num_tiles, splits, 16, 2]
  int table_width, page_size, heads, kv_rank, rot_dim, window, keys_per_split, splits;
  float scale;
};

constexpr int kLatentPad = 8;     // elements between staged rows: operand reads spread over banks

// The wavefronts of a workgroup take consecutive tiles of one entry (where keys are shared
// out, one tile and three empty ones, which only help load) and walk the union of their
// keys together: each block of
// 32 cached rows is staged in LDS once by all of them (16-byte loads, rows that are not
// there as zeros), and both operands come from there: the K operand as 16 bytes of a row,
// the C^T operand as eight 2-byte reads of a column.  A tile with no rows only helps load.
template <int KS, int DB, typename TO>
__global__ __launch_bounds__(4 * kWave) void latent_attention_mfma_kernel(LatentMfmaArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int dl = a.kv_rank + a.rot_dim, P = a.page_size;
  const int stride = dl + kLatentPad;
  bf16_t* k_s = (bf16_t*)lds_raw;                         // [32][stride]
  int* krow_s = (int*)(lds_raw + (size_t)32 * stride * sizeof(bf16_t));   // [32]
  const int waves = blockDim.x / kWave, wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave, r = lane % 16, g = lane / 16;
  const int tile0 = blockIdx.x * waves, tile = tile0 + wave, split = blockIdx.y;
  const int row0 = a.tiles[3 * tile], nrows = a.tiles[3 * tile + 1];
  const int* tab = a.table + (int64_t)a.tiles[3 * tile0 + 2] * a.table_width;
  const bool row_ok = r < nrows;
  const int my_row = row0 + max(0, min(r, nrows - 1));
  const int pos_r = a.positions[my_row / a.heads];
  const int lo_r = a.window > 0 ? max(0, pos_r - a.window + 1) : 0;
  // the keys of the whole workgroup: from the first tile's first token to the last token
  const int pos_first = a.positions[a.tiles[3 * tile0] / a.heads];
  const int lo_t = a.window > 0 ? max(0, pos_first - a.window + 1) : 0;
  int hi_t = pos_first;
  for (int w = 0; w < waves; ++w) {
    const int n = a.tiles[3 * (tile0 + w) + 1];
    if (n > 0) hi_t = max(hi_t, a.positions[(a.tiles[3 * (tile0 + w)] + n - 1) / a.heads]);
  }
  const int k_begin = (lo_t / 32) * 32 + split * a.keys_per_split;
  const int k_end = min(k_begin + a.keys_per_split, hi_t + 1);

  bf16x8_l q[KS];
  const float* qr = a.qa + (int64_t)my_row * dl;
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    const int d0 = 32 * s + 8 * g;
#pragma unroll
    for (int j = 0; j < 8; ++j) q[s][j] = (d0 + j < dl) ? (__bf16)qr[d0 + j] : (__bf16)0.f;
  }
  f32x4_l o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) o[db] = f32x4_l{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const int parts = dl / 8;

  for (int kb = k_begin; kb < k_end; kb += 32) {
    __syncthreads();                      // the block before has been used by everyone
    for (int c = threadIdx.x; c < 32 * parts; c += blockDim.x) {
      const int key = c / parts, part = c % parts;
      const int j = kb + key;
      int page = -1;
      if (j >= lo_t && j <= hi_t) page = tab[j / P];
      const int row = page >= 0 ? page * P + j % P : -1;
      bf16x8_l v;
      if (row >= 0) v = *(const bf16x8_l*)(a.pages + (int64_t)row * dl + part * 8);
      else {
#pragma unroll
        for (int j8 = 0; j8 < 8; ++j8) v[j8] = (__bf16)0.f;
      }
      *(bf16x8_l*)(k_s + key * stride + part * 8) = v;
      if (part == 0) krow_s[key] = row;
    }
    __syncthreads();
    if (__builtin_amdgcn_readfirstlane(nrows) <= 0) continue;   // an empty tile only loads
    f32x4_l st[2];
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
      const bf16_t* kr = k_s + (16 * blk + r) * stride;
      st[blk] = f32x4_l{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const int d0 = 32 * s + 8 * g;
        if (32 * s < dl) {
          bf16x8_l kop;
          if (d0 + 8 <= dl) kop = *(const bf16x8_l*)(kr + d0);
          else {
#pragma unroll
            for (int j8 = 0; j8 < 8; ++j8) kop[j8] = (__bf16)0.f;
          }
          st[blk] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop, q[s], st[blk], 0, 0, 0);
        }
      }
    }
    float sc[8];
    float mx = -INFINITY;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int blk = e / 4, t = e % 4;
      const int key = kb + 16 * blk + 4 * g + t;
      const bool vis = row_ok && krow_s[16 * blk + 4 * g + t] >= 0 && key <= pos_r && key >= lo_r;
      sc[e] = vis ? st[blk][t] * a.scale : -INFINITY;
      mx = fmaxf(mx, sc[e]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    const float m_new = fmaxf(m, mx);
    const float corr = m_new == -INFINITY ? 1.f : expf(m - m_new);
    bf16x8_l pv;
    float psum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float p = sc[e] == -INFINITY ? 0.f : expf(sc[e] - m_new);
      psum += p;
      pv[e] = (__bf16)p;
    }
    psum += __shfl_xor(psum, 16, kWave);
    psum += __shfl_xor(psum, 32, kWave);
    l = l * corr + psum;
    m = m_new;
    const bf16_t* vcol = k_s + (4 * g) * stride + r;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      if (16 * db < a.kv_rank) {
        bf16x8_l vop;
#pragma unroll
        for (int e = 0; e < 8; ++e)
          vop[e] = vcol[(16 * (e / 4) + e % 4) * stride + 16 * db];
        o[db] = o[db] * corr;
        o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop, pv, o[db], 0, 0, 0);
      }
    }
  }
  if (a.splits == 1) {
    if (!row_ok) return;
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    TO* orow = (TO*)a.out + (int64_t)my_row * a.kv_rank;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int d = 16 * db + 4 * g + t;
        if (d < a.kv_rank) orow[d] = from_f32<TO>(o[db][t] * inv);
      }
    return;
  }
  const int64_t slot = ((int64_t)tile * a.splits + split) * 16 + r;
  float* po = a.part_o + slot * a.kv_rank;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int d = 16 * db + 4 * g + t;
      if (d < a.kv_rank) po[d] = o[db][t];
    }
  if (g == 0) {
    a.part_ml[2 * slot] = m;
    a.part_ml[2 * slot + 1] = l;
  }
}

// One workgroup per (tile, row): the shares' results weighted by exp(m_s - max m) and
// divided by the summed weights of their l, shares in index order.  The first wavefront
// turns the shares' statistics into weights (in LDS); then every thread adds its columns
// over the shares, eight loads at a time.
template <typename TO>
__global__ __launch_bounds__(128) void latent_attention_merge_kernel(LatentMfmaArgs a) {
  extern __shared__ float w_s[];            // [splits] weights, then the reciprocal of their sum
  const int tile = blockIdx.x, r = blockIdx.y;
  if (r >= a.tiles[3 * tile + 1]) return;
  const int64_t base = (int64_t)tile * a.splits * 16 + r;
  if (threadIdx.x < kWave) {
    float mx = -INFINITY;
    for (int s = threadIdx.x; s < a.splits; s += kWave)
      mx = fmaxf(mx, a.part_ml[2 * (base + 16 * s)]);
    mx = wave_max(mx);
    float total = 0.f;
    for (int s = threadIdx.x; s < a.splits; s += kWave) {
      const float ms = a.part_ml[2 * (base + 16 * s)];
      const float w = ms == -INFINITY ? 0.f : expf(ms - mx);
      w_s[s] = w;
      total += a.part_ml[2 * (base + 16 * s) + 1] * w;
    }
    total = wave_sum(total);
    if (threadIdx.x == 0) w_s[a.splits] = total > 0.f ? 1.0f / total : 0.f;
  }
  __syncthreads();
  const float inv = w_s[a.splits];
  TO* orow = (TO*)a.out + (int64_t)(a.tiles[3 * tile] + r) * a.kv_rank;
  for (int d = threadIdx.x; d < a.kv_rank; d += blockDim.x) {
    float acc = 0.f;
    int s = 0;
    for (; s + 8 <= a.splits; s += 8) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = a.part_o[(base + 16 * (s + u)) * a.kv_rank + d];
#pragma unroll
      for (int u = 0; u < 8; ++u) acc = fmaf(v[u], w_s[s + u], acc);
    }
    for (; s < a.splits; ++s) acc = fmaf(a.part_o[(base + 16 * s) * a.kv_rank + d], w_s[s], acc);
    orow[d] = from_f32<TO>(acc * inv);
  }
}

template <int KS, int DB>
static int launch_latent_mfma(const LatentMfmaArgs& a, int num_tiles, int waves, int out_type,
                              hipStream_t stream) {
  const int dl = a.kv_rank + a.rot_dim;
  const size_t lds = (size_t)32 * (dl + kLatentPad) * sizeof(bf16_t) + 32 * sizeof(int);
  TS_DISPATCH_TYPE(out_type, TO, {
    hipLaunchKernelGGL((latent_attention_mfma_kernel<KS, DB, TO>),
                       dim3(num_tiles / waves, a.splits), dim3(waves * kWave), lds, stream, a);
    if (a.splits > 1)
      hipLaunchKernelGGL(latent_attention_merge_kernel<TO>, dim3(num_tiles, 16), dim3(128),
                         (size_t)(a.splits + 1) * sizeof(float), stream, a);
  });
  return 0;
}

// 1 if the matrix-core kernel serves these sizes (bfloat16 pages are the caller's to check).
extern "C" int ts_latent_attention_mfma_fits(int kv_rank, int rot_dim) {
  const int dl = kv_rank + rot_dim;
  return dl % 8 == 0 && dl <= 640 && kv_rank <= 512;
}

// `tiles` comes in groups of `waves` (1 or 4) tiles of one entry, a group's last tiles
// possibly empty (0 rows); `num_tiles` counts them all.
extern "C" int ts_latent_attention_mfma(const float* qa, const void* pages, void* out,
                                        int out_type, const int* tiles, int num_tiles, int waves,
                                        const int* positions, const int* table, int table_width,
                                        int page_size, int heads, int kv_rank, int rot_dim,
                                        int window, float scale, int keys_per_split, int splits,
                                        float* part_o, float* part_ml, hipStream_t stream) {
  if (num_tiles <= 0) return 0;
  if (!ts_latent_attention_mfma_fits(kv_rank, rot_dim) || heads <= 0 || page_size <= 0)
    TS_FAIL("latent_attention_mfma: sizes kv_rank=%d rot_dim=%d are not served", kv_rank, rot_dim);
  if (splits < 1 || keys_per_split < 32 || keys_per_split % 32)
    TS_FAIL("latent_attention_mfma: bad split of the keys (%d runs of %d)", splits, keys_per_split);
  if (splits > 1 && (!part_o || !part_ml)) TS_FAIL("latent_attention_mfma: no scratch for the shares");
  if ((waves != 1 && waves != 4) || num_tiles % waves)
    TS_FAIL("latent_attention_mfma: %d tiles in groups of %d", num_tiles, waves);
  if (((uintptr_t)pages & 15) != 0) TS_FAIL("latent_attention_mfma: pages must start on 16 bytes");
  LatentMfmaArgs a{qa, (const bf16_t*)pages, out, tiles, positions, table, part_o, part_ml,
                   table_width, page_size, heads, kv_rank, rot_dim, window, keys_per_split, splits,
                   scale};
  const int dl = kv_rank + rot_dim;
  int rc;
  if (dl <= 96 && kv_rank <= 64) rc = launch_latent_mfma<3, 4>(a, num_tiles, waves, out_type, stream);
  else if (dl <= 320 && kv_rank <= 256) rc = launch_latent_mfma<10, 16>(a, num_tiles, waves, out_type, stream);
  else rc = launch_latent_mfma<20, 32>(a, num_tiles, waves, out_type, stream);
  if (rc) return rc;
  TS_CHECK_LAUNCH("latent_attention_mfma");
  return 0;
}
