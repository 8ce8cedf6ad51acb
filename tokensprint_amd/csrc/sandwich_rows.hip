// Row-wise kernels of layers that norm a sub-layer's output before adding it to the
// residual stream, and of what such models put in front of the stream: a bigram-hashed
// embedding with its norm, the add of a normalised output (alone, or with the next
// sub-layer's norm), the norm with a token shift behind it, and the PolyNorm activation.
// One workgroup per row; every sum, root and product in float32.
//
// Per-request state (the previous token, the previous row of a token shift) lives in
// [slots, ...] arrays indexed by the entry's slot id.  A step reads a request's state for
// the first token of its portion only, and only if that token is not at position 0; the
// workgroup of that first token is also the one that writes the state the portion leaves
// (from the portion's last token), so within a launch every state element is read and then
// written by one thread.
#include "common.h"

__device__ __forceinline__ float inv_rms(float sumsq, int n, float eps) {
  return 1.0f / sqrtf(sumsq / (float)n + eps);
}

// A thread keeps the first kRowItems elements of its share of a row in registers between
// the passes over the row (sum of squares, then the scaled values), so a row of up to
// kRowItems x threads elements is read once; what lies beyond is read again.  A step of
// few rows is a chain of trips to memory and barriers, and this halves the trips.
constexpr int kRowItems = 8;

// Threads for a row of `width` elements: eight elements a thread, 64 to 1024 threads.
static int row_threads(int width) {
  int t = ((width + kRowItems - 1) / kRowItems + 63) / 64 * 64;
  return t < 64 ? 64 : (t > 1024 ? 1024 : t);
}

// ---------------------------------------------------------------- bigram embedding
template <typename TW>
__global__ __launch_bounds__(256) void bigram_embed_kernel(
    const TW* __restrict__ table, const TW* __restrict__ bigram, const float* __restrict__ norm_w,
    const int* __restrict__ ids, const int* __restrict__ positions,
    const int* __restrict__ entry_of_token, const int* __restrict__ q_start,
    const int* __restrict__ slot_ids, int* __restrict__ prev_state, float* __restrict__ out,
    int width, float scale, int buckets, int mul_prev, int mul_cur, float eps) {
  __shared__ float scratch[16];
  __shared__ int row_s;
  const int t = blockIdx.x;
  const int id = ids[t];
  if (threadIdx.x == 0) {
    const int e = entry_of_token[t];
    const int first = q_start[e];
    int prev = -1;
    if (t > first) {
      prev = ids[t - 1];
    } else {
      const int slot = slot_ids[e];
      if (positions[t] > 0) prev = prev_state[slot];
      prev_state[slot] = ids[q_start[e + 1] - 1];
    }
    int row = buckets;
    if (prev >= 0) {
      int64_t v = ((int64_t)prev * mul_prev + (int64_t)id * mul_cur) % buckets;
      if (v < 0) v += buckets;
      row = (int)v;
    }
    row_s = row;
  }
  __syncthreads();
  const TW* er = table + (int64_t)id * width;
  const TW* br = bigram + (int64_t)row_s * width;
  float* o = out + (int64_t)t * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = to_f32(er[i]) * scale + to_f32(br[i]);
    o[i] = v;
    ss += v * v;
  }
  const float r = inv_rms(block_sum(ss, scratch), width, eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) o[i] = o[i] * r * norm_w[i];
}

extern "C" int ts_bigram_embed(const void* table, const void* bigram, int table_type,
                               const float* norm_w, const int* ids, const int* positions,
                               const int* entry_of_token, const int* q_start,
                               const int* slot_ids, int* prev_state, float* out, int num_tokens,
                               int width, float scale, int buckets, int mul_prev, int mul_cur,
                               float eps, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (width <= 0 || buckets <= 0) TS_FAIL("bigram_embed: bad sizes width=%d buckets=%d", width, buckets);
  TS_DISPATCH_TYPE(table_type, TW,
                   hipLaunchKernelGGL(bigram_embed_kernel<TW>, dim3(num_tokens), dim3(256), 0,
                                      stream, (const TW*)table, (const TW*)bigram, norm_w, ids,
                                      positions, entry_of_token, q_start, slot_ids, prev_state,
                                      out, width, scale, buckets, mul_prev, mul_cur, eps));
  TS_CHECK_LAUNCH("bigram_embed");
  return 0;
}

// ---------------------------------------------------------------- add of a normalised output
// resid += delta / rms(delta) * post_w; with NORM also out = resid / rms(resid) * norm_w.
template <typename TO, bool NORM>
__global__ __launch_bounds__(1024) void postnorm_add_kernel(
    float* __restrict__ resid, const float* __restrict__ delta, const float* __restrict__ post_w,
    const float* __restrict__ norm_w, TO* __restrict__ out, int width, float post_eps,
    float norm_eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const int nt = blockDim.x;
  float* x = resid + row * width;
  const float* d = delta + row * width;
  float dc[kRowItems], xc[kRowItems];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < kRowItems; ++k) {
    const int i = threadIdx.x + k * nt;
    dc[k] = i < width ? d[i] : 0.f;
    xc[k] = i < width ? x[i] : 0.f;
    ss += dc[k] * dc[k];
  }
  for (int i = threadIdx.x + kRowItems * nt; i < width; i += nt) ss += d[i] * d[i];
  const float r = inv_rms(block_sum(ss, scratch), width, post_eps);
  float ss2 = 0.f;
#pragma unroll
  for (int k = 0; k < kRowItems; ++k) {
    const int i = threadIdx.x + k * nt;
    if (i < width) {
      xc[k] = xc[k] + dc[k] * r * post_w[i];
      x[i] = xc[k];
      ss2 += xc[k] * xc[k];
    }
  }
  for (int i = threadIdx.x + kRowItems * nt; i < width; i += nt) {
    const float v = x[i] + d[i] * r * post_w[i];
    x[i] = v;
    ss2 += v * v;
  }
  if (NORM) {
    const float r2 = inv_rms(block_sum(ss2, scratch), width, norm_eps);
    TO* o = out + row * width;
#pragma unroll
    for (int k = 0; k < kRowItems; ++k) {
      const int i = threadIdx.x + k * nt;
      if (i < width) o[i] = from_f32<TO>(xc[k] * r2 * norm_w[i]);
    }
    // each thread reads back the elements it wrote itself
    for (int i = threadIdx.x + kRowItems * nt; i < width; i += nt)
      o[i] = from_f32<TO>(x[i] * r2 * norm_w[i]);
  }
}

extern "C" int ts_postnorm_add(float* resid, const float* delta, const float* post_w,
                               float post_eps, const float* norm_w, float norm_eps, void* out,
                               int out_type, int rows, int width, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (width <= 0) TS_FAIL("postnorm_add: bad width %d", width);
  if (norm_w == nullptr) {
    hipLaunchKernelGGL((postnorm_add_kernel<float, false>), dim3(rows), dim3(row_threads(width)),
                       0, stream, resid, delta, post_w, nullptr, nullptr, width, post_eps, 0.f);
  } else {
    TS_DISPATCH_TYPE(out_type, TO,
                     hipLaunchKernelGGL((postnorm_add_kernel<TO, true>), dim3(rows),
                                        dim3(row_threads(width)), 0, stream, resid, delta, post_w,
                                        norm_w, (TO*)out, width, post_eps, norm_eps));
  }
  TS_CHECK_LAUNCH("postnorm_add");
  return 0;
}

// ---------------------------------------------------------------- norm and token shift
// h_t = resid_t / rms(resid_t) * w;  out_t = h_t + (h_(t-1) - h_t) * shift.
// h_(t-1) is recomputed from the row before inside a portion, read from the request's
// state at a portion's first token, and zero at position 0.
template <typename TO>
__global__ __launch_bounds__(1024) void norm_token_shift_kernel(
    const float* __restrict__ resid, const float* __restrict__ norm_w,
    const float* __restrict__ shift_w, float* __restrict__ state, TO* __restrict__ out,
    const int* __restrict__ positions, const int* __restrict__ entry_of_token,
    const int* __restrict__ q_start, const int* __restrict__ slot_ids, int width, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, nt = blockDim.x;
  const int e = entry_of_token[t];
  const int first = q_start[e], last = q_start[e + 1] - 1;
  const bool is_first = t == first;
  const bool from_state = is_first && positions[t] > 0;
  const bool other_last = is_first && last != t;
  const float* x = resid + (int64_t)t * width;
  const float* xp = resid + (int64_t)(t - 1) * width;
  const float* xl = resid + (int64_t)last * width;
  float* st = state + (int64_t)slot_ids[e] * width;
  // the row, and the one other row this workgroup needs (the row before, or the portion's
  // last row whose norm goes into the state), both kept in registers
  const float* y = !is_first ? xp : xl;
  const bool need_y = !is_first || other_last;
  float xc[kRowItems], yc[kRowItems];
  float ss = 0.f, ssy = 0.f;
#pragma unroll
  for (int k = 0; k < kRowItems; ++k) {
    const int i = threadIdx.x + k * nt;
    xc[k] = i < width ? x[i] : 0.f;
    yc[k] = (need_y && i < width) ? y[i] : 0.f;
    ss += xc[k] * xc[k];
    ssy += yc[k] * yc[k];
  }
  for (int i = threadIdx.x + kRowItems * nt; i < width; i += nt) {
    ss += x[i] * x[i];
    if (need_y) ssy += y[i] * y[i];
  }
  const float r = inv_rms(block_sum(ss, scratch), width, eps);
  float ry = r;
  if (need_y) ry = inv_rms(block_sum(ssy, scratch), width, eps);
  TO* o = out + (int64_t)t * width;
  auto finish = [&](int i, float xv, float yv) {
    const float w = norm_w[i];
    const float h = xv * r * w;
    float prev = 0.f;
    if (!is_first) prev = yv * ry * w;
    else if (from_state) prev = st[i];
    o[i] = from_f32<TO>(h + (prev - h) * shift_w[i]);
    if (is_first) st[i] = other_last ? yv * ry * w : h;
  };
#pragma unroll
  for (int k = 0; k < kRowItems; ++k) {
    const int i = threadIdx.x + k * nt;
    if (i < width) finish(i, xc[k], yc[k]);
  }
  for (int i = threadIdx.x + kRowItems * nt; i < width; i += nt)
    finish(i, x[i], need_y ? y[i] : 0.f);
}

extern "C" int ts_norm_token_shift(const float* resid, const float* norm_w, float eps,
                                   const float* shift_w, float* state, void* out, int out_type,
                                   const int* positions, const int* entry_of_token,
                                   const int* q_start, const int* slot_ids, int num_tokens,
                                   int width, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (width <= 0) TS_FAIL("norm_token_shift: bad width %d", width);
  TS_DISPATCH_TYPE(out_type, TO,
                   hipLaunchKernelGGL(norm_token_shift_kernel<TO>, dim3(num_tokens),
                                      dim3(row_threads(width)), 0, stream, resid, norm_w, shift_w,
                                      state, (TO*)out, positions, entry_of_token, q_start,
                                      slot_ids, width, eps));
  TS_CHECK_LAUNCH("norm_token_shift");
  return 0;
}

// ---------------------------------------------------------------- PolyNorm
// out = a z/rms(z) + b z^2/rms(z^2) + c z^3/rms(z^3) + e, powers element by element.
template <typename TO>
__global__ __launch_bounds__(1024) void polynorm_kernel(const float* __restrict__ z,
                                                        const float* __restrict__ coef,
                                                        TO* __restrict__ out, int width,
                                                        float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const int nt = blockDim.x;
  const float* x = z + row * width;
  float zc[kRowItems];
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  auto add = [&](float v) {
    const float v2 = v * v, v3 = v2 * v;
    s2 += v2;
    s4 += v2 * v2;
    s6 += v3 * v3;
  };
#pragma unroll
  for (int k = 0; k < kRowItems; ++k) {
    const int i = threadIdx.x + k * nt;
    zc[k] = i < width ? x[i] : 0.f;
    add(zc[k]);
  }
  for (int i = threadIdx.x + kRowItems * nt; i < width; i += nt) add(x[i]);
  const float r1 = inv_rms(block_sum(s2, scratch), width, eps);
  const float r2 = inv_rms(block_sum(s4, scratch), width, eps);
  const float r3 = inv_rms(block_sum(s6, scratch), width, eps);
  const float a = coef[0], b = coef[1], c = coef[2], e = coef[3];
  TO* o = out + row * width;
  auto value = [&](float v) {
    const float v2 = v * v;
    return a * (v * r1) + b * (v2 * r2) + c * (v2 * v * r3) + e;
  };
#pragma unroll
  for (int k = 0; k < kRowItems; ++k) {
    const int i = threadIdx.x + k * nt;
    if (i < width) o[i] = from_f32<TO>(value(zc[k]));
  }
  for (int i = threadIdx.x + kRowItems * nt; i < width; i += nt) o[i] = from_f32<TO>(value(x[i]));
}

extern "C" int ts_polynorm(const float* z, const float* coef, void* out, int out_type, int rows,
                           int width, float eps, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (width <= 0) TS_FAIL("polynorm: bad width %d", width);
  TS_DISPATCH_TYPE(out_type, TO,
                   hipLaunchKernelGGL(polynorm_kernel<TO>, dim3(rows), dim3(row_threads(width)), 0,
                                      stream, z, coef, (TO*)out, width, eps));
  TS_CHECK_LAUNCH("polynorm");
  return 0;
}
