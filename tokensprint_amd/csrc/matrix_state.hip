// Kernels of the mixers that keep a matrix per head and request: linear attention with a
// decay, and the gated delta rule.  One recurrence serves both:
//
//   S <- g S                    g: a number per head (fixed, or one per token), or one per
//                               row of S (a decay per key channel)
//   u = v                       (linear attention)
//   u = beta (v - S^T k)        (delta rule)
//   S <- S + k u^T;   o = S^T q
//
// S is N x P (key channels x value channels), float32, zero at a sequence's start, kept in
// the request's state slot between steps.  All arithmetic in float32.  Beside it: the
// preparation of the delta rule's operands (unit vectors, beta, decays) and the norm with a
// gate behind the recurrence.
//
// A request's state is read only where a portion does not start at position 0, and is
// written once a portion, by the thread that owns the element.
#include "common.h"

struct BatchView {
  const int* positions;       // [T]
  const int* entry_of_token;  // [T]
  const int* q_start;         // [B + 1]
  const int* slot_ids;        // [B]
};

__device__ __forceinline__ float sigmoid_f(float v) { return 1.0f / (1.0f + expf(-v)); }
__device__ __forceinline__ float silu_f(float v) { return v / (1.0f + expf(-v)); }
__device__ __forceinline__ float softplus_f(float v) { return v > 20.f ? v : log1pf(expf(v)); }

// ---------------------------------------------------------------- recurrence
struct RecurrenceArgs {
  const float* x;        // [T, ld]: q (kv_heads*N) at q_col, k at k_col, v (heads*P) at v_col
  const float* decay;    // [heads]: the fixed decays, or null
  const float* gates;    // [T, ldg]: beta (heads) | g (heads, or heads*N), or null
  float* state;          // [slots, heads, N, P]
  float* out;            // [T, heads*P]
  BatchView b;
  int ld, q_col, k_col, v_col, ldg, heads, kv_heads, N, P, silu;
};

constexpr int kRecSlices = 8;              // lanes that share a column's dot products
constexpr int kRecThreads = 128;
constexpr int kRecPerThread = 4;           // columns a thread owns
constexpr int kRecBlockCols = kRecThreads / kRecSlices * kRecPerThread;   // 64
constexpr int kRecStage = 16;              // tokens staged in LDS at a time

// A workgroup serves one (entry, head, 64 columns of P) and walks the entry's tokens in
// order.  Thread (cg, s) = (tid / 8, tid % 8) keeps rows s, s + 8, ... of four columns in
// registers; sixteen tokens' q, k, the workgroup's columns of v, and the gates are staged in
// LDS by all threads together; a column's dot products over the rows are added over the
// eight lanes that share it, in one fixed butterfly.
template <int NI, bool DELTA, bool PER_ROW>
__global__ __launch_bounds__(kRecThreads) void recurrence_kernel(RecurrenceArgs a) {
  extern __shared__ float lds[];
  const int N = a.N;
  float* q_s = lds;                                  // [stage][N]
  float* k_s = q_s + kRecStage * N;                  // [stage][N]
  float* g_s = k_s + kRecStage * N;                  // [stage][N] (PER_ROW) or [stage]
  float* v_s = g_s + kRecStage * (PER_ROW ? N : 1);  // [stage][64]
  float* b_s = v_s + kRecStage * kRecBlockCols;      // [stage]: beta
  const int h = blockIdx.x, e = blockIdx.y;
  const int s = threadIdx.x % kRecSlices, cg = threadIdx.x / kRecSlices;
  const int col0 = blockIdx.z * kRecBlockCols;
  const int p0 = col0 + cg * kRecPerThread;
  const int hk = h / (a.heads / a.kv_heads);
  const int first = a.b.q_start[e], end = a.b.q_start[e + 1];
  float* st = a.state + ((int64_t)a.b.slot_ids[e] * a.heads + h) * N * a.P;
  const bool fresh = a.b.positions[first] == 0;
  float S[NI][kRecPerThread];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int n = s + kRecSlices * i;
#pragma unroll
    for (int c = 0; c < kRecPerThread; ++c)
      S[i][c] = (!fresh && n < N && p0 + c < a.P) ? st[(int64_t)n * a.P + p0 + c] : 0.f;
  }
  const float fixed_decay = a.decay ? a.decay[h] : 1.f;
  const int inner = a.heads * a.P;

  for (int t0 = first; t0 < end; t0 += kRecStage) {
    const int nt = min(kRecStage, end - t0);
    __syncthreads();                                  // the stage before has been walked
    for (int i = threadIdx.x; i < nt * N; i += kRecThreads) {
      const int tt = i / N, n = i % N;
      const float* row = a.x + (int64_t)(t0 + tt) * a.ld;
      float qv = row[a.q_col + hk * N + n], kv = row[a.k_col + hk * N + n];
      if (a.silu) qv = silu_f(qv), kv = silu_f(kv);
      q_s[i] = qv;
      k_s[i] = kv;
      if (PER_ROW) g_s[i] = a.gates[(int64_t)(t0 + tt) * a.ldg + a.heads + h * N + n];
    }
    for (int i = threadIdx.x; i < kRecStage * kRecBlockCols; i += kRecThreads) {
      const int tt = i / kRecBlockCols, c = i % kRecBlockCols;
      float v = 0.f;
      if (tt < nt && col0 + c < a.P) {
        v = a.x[(int64_t)(t0 + tt) * a.ld + a.v_col + h * a.P + col0 + c];
        if (a.silu) v = silu_f(v);
      }
      v_s[i] = v;
    }
    if (threadIdx.x < nt) {
      const float* gr = a.gates ? a.gates + (int64_t)(t0 + threadIdx.x) * a.ldg : nullptr;
      if (DELTA) b_s[threadIdx.x] = gr[h];
      if (!PER_ROW) g_s[threadIdx.x] = gr ? gr[a.heads + h] : fixed_decay;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      float u[kRecPerThread], acc[kRecPerThread];
#pragma unroll
      for (int c = 0; c < kRecPerThread; ++c) u[c] = v_s[tt * kRecBlockCols + cg * kRecPerThread + c];
      const float g_all = PER_ROW ? 1.f : g_s[tt];
      if (DELTA) {
        float pred[kRecPerThread];
#pragma unroll
        for (int c = 0; c < kRecPerThread; ++c) pred[c] = 0.f;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          const int n = s + kRecSlices * i;
          const float kv = n < N ? k_s[tt * N + n] : 0.f;
          const float g = PER_ROW ? (n < N ? g_s[tt * N + n] : 1.f) : g_all;
#pragma unroll
          for (int c = 0; c < kRecPerThread; ++c) {
            S[i][c] *= g;
            pred[c] = fmaf(S[i][c], kv, pred[c]);
          }
        }
        const float beta = b_s[tt];
#pragma unroll
        for (int c = 0; c < kRecPerThread; ++c) {
          pred[c] += __shfl_xor(pred[c], 1, kWave);
          pred[c] += __shfl_xor(pred[c], 2, kWave);
          pred[c] += __shfl_xor(pred[c], 4, kWave);
          u[c] = beta * (u[c] - pred[c]);
        }
      }
#pragma unroll
      for (int c = 0; c < kRecPerThread; ++c) acc[c] = 0.f;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int n = s + kRecSlices * i;
        const float kv = n < N ? k_s[tt * N + n] : 0.f;
        const float qv = n < N ? q_s[tt * N + n] : 0.f;
#pragma unroll
        for (int c = 0; c < kRecPerThread; ++c) {
          if (DELTA) S[i][c] = fmaf(kv, u[c], S[i][c]);
          else S[i][c] = fmaf(g_all, S[i][c], kv * u[c]);
          acc[c] = fmaf(S[i][c], qv, acc[c]);
        }
      }
#pragma unroll
      for (int c = 0; c < kRecPerThread; ++c) {
        acc[c] += __shfl_xor(acc[c], 1, kWave);
        acc[c] += __shfl_xor(acc[c], 2, kWave);
        acc[c] += __shfl_xor(acc[c], 4, kWave);
        if (s == 0 && p0 + c < a.P) a.out[(int64_t)(t0 + tt) * inner + h * a.P + p0 + c] = acc[c];
      }
    }
  }
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int n = s + kRecSlices * i;
#pragma unroll
    for (int c = 0; c < kRecPerThread; ++c)
      if (n < N && p0 + c < a.P) st[(int64_t)n * a.P + p0 + c] = S[i][c];
  }
}

template <int NI>
static void launch_recurrence(const RecurrenceArgs& a, int num_entries, bool delta, bool per_row,
                              hipStream_t stream) {
  const dim3 grid(a.heads, num_entries, (a.P + kRecBlockCols - 1) / kRecBlockCols);
  const dim3 block(kRecThreads);
  const size_t lds = (size_t)kRecStage * (2 * a.N + (per_row ? a.N : 1) + kRecBlockCols + 1) *
                     sizeof(float);
  if (delta && per_row)
    hipLaunchKernelGGL((recurrence_kernel<NI, true, true>), grid, block, lds, stream, a);
  else if (delta)
    hipLaunchKernelGGL((recurrence_kernel<NI, true, false>), grid, block, lds, stream, a);
  else
    hipLaunchKernelGGL((recurrence_kernel<NI, false, false>), grid, block, lds, stream, a);
}

// x [T, ld] float32 holds q, k (kv_heads x N each) and v (heads x P) at the given columns
// (`silu`: their SiLU is taken as they are read).  `decay` [heads]: fixed decays, or null and
// `gates` [T, ldg] holds beta (heads; read by the delta rule only) and then the decays, one
// per head or (`per_row`) one per head and row of S.  out [T, heads*P].
extern "C" int ts_linear_recurrence(const float* x, int ld, int q_col, int k_col, int v_col,
                                    const float* decay, const float* gates, int ldg, float* state,
                                    float* out, const int* positions, const int* entry_of_token,
                                    const int* q_start, const int* slot_ids, int num_tokens,
                                    int num_entries, int heads, int kv_heads, int N, int P,
                                    int silu, int delta, int per_row, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || N <= 0 || P <= 0)
    TS_FAIL("linear_recurrence: bad sizes heads=%d kv_heads=%d dim=%d vdim=%d", heads, kv_heads, N, P);
  if (N > kRecSlices * 32)
    TS_FAIL("linear_recurrence: %d key channels, at most %d are built", N, kRecSlices * 32);
  if (q_col < 0 || k_col < 0 || v_col < 0 || q_col + kv_heads * N > ld || k_col + kv_heads * N > ld ||
      v_col + heads * P > ld)
    TS_FAIL("linear_recurrence: columns outside the rows (ld=%d)", ld);
  if ((decay != nullptr) == (gates != nullptr))
    TS_FAIL("linear_recurrence: either fixed decays or gates per token");
  if ((delta || per_row) && !gates) TS_FAIL("linear_recurrence: the delta rule needs gates per token");
  if (per_row && !delta) TS_FAIL("linear_recurrence: decays per row are built for the delta rule");
  if (gates && ldg < heads + (per_row ? heads * N : heads))
    TS_FAIL("linear_recurrence: gates of %d columns are too few", ldg);
  RecurrenceArgs a{x, decay, gates, state, out,
                   BatchView{positions, entry_of_token, q_start, slot_ids},
                   ld, q_col, k_col, v_col, ldg, heads, kv_heads, N, P, silu};
  const int ni = (N + kRecSlices - 1) / kRecSlices;
  if (ni <= 2) launch_recurrence<2>(a, num_entries, delta, per_row, stream);
  else if (ni <= 4) launch_recurrence<4>(a, num_entries, delta, per_row, stream);
  else if (ni <= 8) launch_recurrence<8>(a, num_entries, delta, per_row, stream);
  else if (ni <= 16) launch_recurrence<16>(a, num_entries, delta, per_row, stream);
  else launch_recurrence<32>(a, num_entries, delta, per_row, stream);
  TS_CHECK_LAUNCH("linear_recurrence");
  return 0;
}

// ---------------------------------------------------------------- the delta rule's operands
// In place on qkv [T, ld]: every q and k head (kv_heads x N each, q from column 0, k behind
// it) becomes x / sqrt(sum(x^2) + 1e-6), q also times N^-1/2.  Into gates [T, ldg]:
// beta = sigmoid(proj[beta_col + h]); g = exp(-exp(A_log[h]) softplus(z[z_col + j] +
// dt_bias[j])), j over heads or (`per_row`) over heads x N.
__global__ __launch_bounds__(256) void delta_gates_kernel(
    float* __restrict__ qkv, int ld, const float* __restrict__ proj, int ldp, int beta_col,
    const float* __restrict__ z, int ldz, int z_col, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, float* __restrict__ gates, int ldg, int heads,
    int kv_heads, int N, int per_row) {
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave, waves = blockDim.x / kWave;
  for (int u = wave; u < 2 * kv_heads; u += waves) {
    float* v = qkv + t * ld + (int64_t)u * N;
    float ss = 0.f;
    for (int i = lane; i < N; i += kWave) ss = fmaf(v[i], v[i], ss);
    ss = wave_sum(ss);
    const float r = (1.0f / sqrtf(ss + 1e-6f)) * (u < kv_heads ? 1.0f / sqrtf((float)N) : 1.f);
    for (int i = lane; i < N; i += kWave) v[i] *= r;
  }
  const int ng = per_row ? heads * N : heads;
  for (int c = threadIdx.x; c < heads + ng; c += blockDim.x) {
    float out;
    if (c < heads) {
      out = sigmoid_f(proj[t * ldp + beta_col + c]);
    } else {
      const int j = c - heads, h = per_row ? j / N : j;
      out = expf(-expf(a_log[h]) * softplus_f(z[t * ldz + z_col + j] + dt_bias[j]));
    }
    gates[t * ldg + c] = out;
  }
}

extern "C" int ts_delta_gates(float* qkv, int ld, const float* proj, int ldp, int beta_col,
                              const float* z, int ldz, int z_col, const float* a_log,
                              const float* dt_bias, float* gates, int ldg, int rows, int heads,
                              int kv_heads, int N, int per_row, hipStream_t stream) {
  if (rows <= 0) return 0;
  const int ng = per_row ? heads * N : heads;
  if (heads <= 0 || kv_heads <= 0 || N <= 0 || 2 * kv_heads * N > ld || beta_col < 0 ||
      beta_col + heads > ldp || z_col < 0 || z_col + ng > ldz || ldg < heads + ng)
    TS_FAIL("delta_gates: sizes do not fit (heads=%d kv_heads=%d dim=%d)", heads, kv_heads, N);
  hipLaunchKernelGGL(delta_gates_kernel, dim3(rows), dim3(256), 0, stream, qkv, ld, proj, ldp,
                     beta_col, z, ldz, z_col, a_log, dt_bias, gates, ldg, heads, kv_heads, N,
                     per_row);
  TS_CHECK_LAUNCH("delta_gates");
  return 0;
}

// ---------------------------------------------------------------- norm and gate
// Each of `groups` equal parts of a row of y is divided by its root mean square, weighed by
// w (w_len values: one per column of a part, shared by the parts, or one per column of the
// row) and multiplied by act(gate[gate_col + column]); act: 0 sigmoid, 1 SiLU.
// One wavefront per (row, part).
template <typename TO>
__global__ __launch_bounds__(256) void norm_gate_kernel(
    const float* __restrict__ y, const float* __restrict__ gate, int ldgate, int gate_col,
    const float* __restrict__ w, int w_len, TO* __restrict__ out, int64_t rows, int inner,
    int groups, int act, float eps) {
  const int64_t unit = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (unit >= rows * groups) return;
  const int lane = threadIdx.x % kWave;
  const int64_t t = unit / groups;
  const int grp = (int)(unit % groups), size = inner / groups;
  const float* yr = y + t * inner + grp * size;
  const float* gr = gate + t * ldgate + gate_col + grp * size;
  const float* wr = w + (w_len == size ? 0 : grp * size);
  float ss = 0.f;
  for (int i = lane; i < size; i += kWave) ss = fmaf(yr[i], yr[i], ss);
  const float r = 1.0f / sqrtf(wave_sum(ss) / (float)size + eps);
  TO* o = out + t * inner + grp * size;
  for (int i = lane; i < size; i += kWave) {
    const float g = gr[i];
    o[i] = from_f32<TO>(yr[i] * r * wr[i] * (act == 0 ? sigmoid_f(g) : silu_f(g)));
  }
}

extern "C" int ts_norm_gate(const float* y, const float* gate, int ldgate, int gate_col,
                            const float* w, int w_len, void* out, int out_type, int rows,
                            int inner, int groups, int act, float eps, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (inner <= 0 || groups <= 0 || inner % groups || gate_col < 0 || gate_col + inner > ldgate ||
      (w_len != inner && w_len != inner / groups) || (act != 0 && act != 1))
    TS_FAIL("norm_gate: bad sizes inner=%d groups=%d weight=%d gate columns %d..%d of %d", inner,
            groups, w_len, gate_col, gate_col + inner, ldgate);
  const int64_t units = (int64_t)rows * groups;
  TS_DISPATCH_TYPE(out_type, TO,
                   hipLaunchKernelGGL(norm_gate_kernel<TO>, dim3((unsigned)((units + 3) / 4)),
                                      dim3(256), 0, stream, y, gate, ldgate, gate_col, w, w_len,
                                      (TO*)out, (int64_t)rows, inner, groups, act, eps));
  TS_CHECK_LAUNCH("norm_gate");
  return 0;
}
