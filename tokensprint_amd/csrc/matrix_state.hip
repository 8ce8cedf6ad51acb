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
  const int* chunks;        // [num_chunks, 3]: first token, one past the last, entry
  const int* entry_chunks;  // [B + 1]: the chunks of entry e are [entry_chunks[e], entry_chunks[e+1])
  float* chunk_state;       // [num_chunks, heads, N, P]: local contribution, then start state
  float* chunk_decay;       // [num_chunks, heads]
};

// Without the delta rule the recurrence is linear in S, and a long portion is cut into
// chunks of 64 tokens that run side by side, in three launches: every chunk's recurrence
// from an empty state (its own contribution and the product of its decays, kRecLocal); per
// entry, the state in front of every chunk, one after the other, and the state the portion
// leaves (combine); every chunk once more from its true start state, now writing o
// (kRecOutput).  Twice the arithmetic, a sixty-fourth of the chain.
constexpr int kRecWhole = 0, kRecLocal = 1, kRecOutput = 2;

constexpr int kRecThreads = 128;
constexpr int kRecStage = 16;              // tokens staged in LDS at a time

// Sum over the eight or sixteen neighbouring lanes that share a column; every one of them
// gets it.  Two exchanges inside a quad, one with the mirrored lane of the eight and one with
// the lane eight further in the row of sixteen, all in the
// vector pipeline (a shuffle through LDS costs a round trip each, on the recurrence's chain).
template <int SL>
__device__ __forceinline__ float sum_slices(float v) {
  static_assert(SL == 8 || SL == 16, "eight or sixteen lanes share a column");
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, true));
  if (SL == 16)      // the other eight of a row of sixteen: rotated by eight
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, true));
  return v;
}

template <int NI>
__device__ __forceinline__ void read_rows(const float* p, float (&r)[NI]) {
  if constexpr (NI % 4 == 0) {
#pragma unroll
    for (int j = 0; j < NI / 4; ++j) {
      const float4 v = reinterpret_cast<const float4*>(p)[j];
      r[4 * j] = v.x, r[4 * j + 1] = v.y, r[4 * j + 2] = v.z, r[4 * j + 3] = v.w;
    }
  } else {
#pragma unroll
    for (int j = 0; j < NI; ++j) r[j] = p[j];
  }
}

// A workgroup serves one (entry, head, 128 / SL x CPT columns of P) and walks the entry's
// tokens in order.  Thread (cg, s) = (tid / SL, tid % SL) keeps rows [s NI, (s + 1) NI) of CPT
// columns in registers; a column's dot products over the rows are added over the SL lanes
// that share it.  Sixteen tokens' q, k, the workgroup's columns of v, and the gates are
// staged in one of two LDS buffers (rows padded to SL NI, so a thread's rows come in 16-byte
// reads) while the sixteen before them are walked.  A token's time is the chain of its
// multiply-adds in one wavefront, so a long portion of few entries takes sixteen lanes a
// column and one column a thread (half the rows a lane, twice the wavefronts), a step of
// many entries eight lanes and four columns (its states stream in wider rows).
template <int NI, int CPT, int SL, bool DELTA, bool PER_ROW, int MODE = kRecWhole>
__global__ __launch_bounds__(kRecThreads) void recurrence_kernel(RecurrenceArgs a) {
  constexpr int kRecSlices = SL, kRecGroups = kRecThreads / SL;
  constexpr int EPT = kRecStage * SL * NI / kRecThreads;   // elements of q a thread stages
  extern __shared__ __align__(16) float lds[];
  constexpr int NP = kRecSlices * NI;                // padded rows
  // a token's rows in LDS: the eight slices' runs of NI rows, 16 bytes between them, so that
  // the eight 16-byte reads of an instruction fall into different banks
  constexpr int SP = NI + 4, LP = kRecSlices * SP;
  constexpr int BC = kRecGroups * CPT;               // columns of the workgroup
  constexpr int kQ = 0, kK = kRecStage * LP, kG = 2 * kRecStage * LP;
  constexpr int kV = kG + kRecStage * (PER_ROW ? LP : 1);
  constexpr int kB = kV + kRecStage * BC;
  constexpr int kBuf = (kB + kRecStage + 3) / 4 * 4;
  constexpr int VPT = kRecStage * BC / kRecThreads;  // values of v a thread stages
  const int N = a.N;
  const int h = blockIdx.x;
  const int s = threadIdx.x % kRecSlices, cg = threadIdx.x / kRecSlices;
  const int col0 = blockIdx.z * BC;
  const int p0 = col0 + cg * CPT;
  const int hk = h / (a.heads / a.kv_heads);
  int first, end, e;
  if (MODE == kRecWhole) {
    e = blockIdx.y;
    first = a.b.q_start[e];
    end = a.b.q_start[e + 1];
  } else {
    first = a.chunks[3 * blockIdx.y];
    end = a.chunks[3 * blockIdx.y + 1];
    e = a.chunks[3 * blockIdx.y + 2];
  }
  float* st = MODE == kRecWhole
      ? a.state + ((int64_t)a.b.slot_ids[e] * a.heads + h) * N * a.P
      : a.chunk_state + ((int64_t)blockIdx.y * a.heads + h) * N * a.P;
  const bool fresh = MODE == kRecLocal || (MODE == kRecWhole && a.b.positions[first] == 0);
  float total_decay = 1.f;
  float S[NI][CPT];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int n = s * NI + i;
#pragma unroll
    for (int c = 0; c < CPT; ++c)
      S[i][c] = (!fresh && n < N && p0 + c < a.P) ? st[(int64_t)n * a.P + p0 + c] : 0.f;
  }
  const float fixed_decay = a.decay ? a.decay[h] : 1.f;
  const int inner = a.heads * a.P;
  for (int i = threadIdx.x; i < 2 * kBuf; i += kRecThreads) lds[i] = 0.f;   // the rows' padding
  __syncthreads();

  // a stage's operands: from memory into registers (fetch), from there into a buffer (commit)
  float pq[EPT], pk[EPT], pg[PER_ROW ? EPT : 1], pv[VPT], pbeta = 0.f, pgate = 1.f;
  auto fetch = [&](int t0) {
    const int nt = min(kRecStage, end - t0);
    // (element j of a thread is row i % NP of token i / NP in the padded layout: NP is a
    // power of two, so no division by a size only known at run time)
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      const int i = j * kRecThreads + threadIdx.x;
      const int tt = i / NP, n = i % NP;
      pq[j] = pk[j] = 0.f;
      if (PER_ROW) pg[j] = 0.f;
      if (tt < nt && n < N) {
        const float* row = a.x + (int64_t)(t0 + tt) * a.ld;
        pq[j] = row[a.q_col + hk * N + n];
        pk[j] = row[a.k_col + hk * N + n];
        if (PER_ROW) pg[j] = a.gates[(int64_t)(t0 + tt) * a.ldg + a.heads + h * N + n];
      }
    }
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      const int i = j * kRecThreads + threadIdx.x;
      const int tt = i / BC, c = i % BC;
      pv[j] = (tt < nt && col0 + c < a.P)
          ? a.x[(int64_t)(t0 + tt) * a.ld + a.v_col + h * a.P + col0 + c] : 0.f;
    }
    if (threadIdx.x < nt) {
      const float* gr = a.gates ? a.gates + (int64_t)(t0 + threadIdx.x) * a.ldg : nullptr;
      if (DELTA) pbeta = gr[h];
      if (!PER_ROW) pgate = gr ? gr[a.heads + h] : fixed_decay;
    }
  };
  auto commit = [&](float* buf) {
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      const int i = j * kRecThreads + threadIdx.x;       // = token * NP + row, padding included
      const int at = (i / NP) * LP + (i % NP) / NI * SP + i % NI;
      buf[kQ + at] = a.silu ? silu_f(pq[j]) : pq[j];
      buf[kK + at] = a.silu ? silu_f(pk[j]) : pk[j];
      if (PER_ROW) buf[kG + at] = pg[j];
    }
#pragma unroll
    for (int j = 0; j < VPT; ++j)
      buf[kV + j * kRecThreads + threadIdx.x] = a.silu ? silu_f(pv[j]) : pv[j];
    if (threadIdx.x < kRecStage) {
      if (DELTA) buf[kB + threadIdx.x] = pbeta;
      if (!PER_ROW) buf[kG + threadIdx.x] = pgate;
    }
  };

  fetch(first);
  commit(lds);
  __syncthreads();
  int which = 0;
  for (int t0 = first; t0 < end; t0 += kRecStage, which ^= 1) {
    const int nt = min(kRecStage, end - t0);
    const bool more = t0 + kRecStage < end;
    if (more) fetch(t0 + kRecStage);
    const float* buf = lds + which * kBuf;
    for (int tt = 0; tt < nt; ++tt) {
      float kr[NI], qr[NI], u[CPT], acc[CPT];
      read_rows<NI>(buf + kK + tt * LP + s * SP, kr);
      if (MODE != kRecLocal) read_rows<NI>(buf + kQ + tt * LP + s * SP, qr);   // one trip to LDS a token
#pragma unroll
      for (int c = 0; c < CPT; ++c) u[c] = buf[kV + tt * BC + cg * CPT + c];
      const float g_all = PER_ROW ? 1.f : buf[kG + tt];
      if (DELTA) {
        float gr[NI];
        if constexpr (PER_ROW) read_rows<NI>(buf + kG + tt * LP + s * SP, gr);
        float pred[CPT][2];
#pragma unroll
        for (int c = 0; c < CPT; ++c) pred[c][0] = pred[c][1] = 0.f;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          const float g = PER_ROW ? gr[i] : g_all;
#pragma unroll
          for (int c = 0; c < CPT; ++c) {
            S[i][c] *= g;
            pred[c][i & 1] = fmaf(S[i][c], kr[i], pred[c][i & 1]);
          }
        }
        const float beta = buf[kB + tt];
#pragma unroll
        for (int c = 0; c < CPT; ++c) u[c] = beta * (u[c] - sum_slices<SL>(pred[c][0] + pred[c][1]));
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
          for (int c = 0; c < CPT; ++c) S[i][c] = fmaf(kr[i], u[c], S[i][c]);
      } else {
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
          for (int c = 0; c < CPT; ++c) S[i][c] = fmaf(g_all, S[i][c], kr[i] * u[c]);
      }
      if (MODE == kRecLocal) {
        total_decay *= g_all;
        continue;
      }
#pragma unroll
      for (int c = 0; c < CPT; ++c) {
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int i = 0; i < NI; i += 2) {
          a0 = fmaf(S[i][c], qr[i], a0);
          a1 = fmaf(S[i + 1][c], qr[i + 1], a1);
        }
        acc[c] = sum_slices<SL>(a0 + a1);
        if (s == 0 && p0 + c < a.P) a.out[(int64_t)(t0 + tt) * inner + h * a.P + p0 + c] = acc[c];
      }
    }
    if (more) commit(lds + (which ^ 1) * kBuf);
    __syncthreads();
  }
  if (MODE == kRecOutput) return;
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int n = s * NI + i;
#pragma unroll
    for (int c = 0; c < CPT; ++c)
      if (n < N && p0 + c < a.P) st[(int64_t)n * a.P + p0 + c] = S[i][c];
  }
  if (MODE == kRecLocal && blockIdx.z == 0 && threadIdx.x == 0)
    a.chunk_decay[(int64_t)blockIdx.y * a.heads + h] = total_decay;
}

// A thread per element of S and (head, entry): walks the entry's chunks in order.
// chunk_state[c] holds the chunk's own contribution and receives the state in front of the
// chunk; the state behind the last chunk goes to the request's slot.
__global__ __launch_bounds__(256) void recurrence_combine_kernel(RecurrenceArgs a) {
  const int h = blockIdx.x, e = blockIdx.y;
  const int idx = blockIdx.z * blockDim.x + threadIdx.x;
  const int size = a.N * a.P;
  if (idx >= size) return;
  float* st = a.state + ((int64_t)a.b.slot_ids[e] * a.heads + h) * size;
  float S = a.b.positions[a.b.q_start[e]] == 0 ? 0.f : st[idx];
  for (int c = a.entry_chunks[e]; c < a.entry_chunks[e + 1]; ++c) {
    float* cs = a.chunk_state + ((int64_t)c * a.heads + h) * size;
    const float local = cs[idx];
    cs[idx] = S;
    S = fmaf(a.chunk_decay[(int64_t)c * a.heads + h], S, local);
  }
  st[idx] = S;
}

template <int NI, int CPT>
static void launch_recurrence_chunked(const RecurrenceArgs& a, int num_entries, int num_chunks,
                                      hipStream_t stream) {
  constexpr int SL = 8, LP = SL * (NI + 4), BC = kRecThreads / SL * CPT;
  const dim3 grid(a.heads, num_chunks, (a.P + BC - 1) / BC);
  const int buf = (kRecStage * (2 * LP + 1 + BC + 1) + 3) / 4 * 4;
  const size_t lds = (size_t)2 * buf * sizeof(float);
  hipLaunchKernelGGL((recurrence_kernel<NI, CPT, 8, false, false, kRecLocal>), grid,
                     dim3(kRecThreads), lds, stream, a);
  hipLaunchKernelGGL(recurrence_combine_kernel, dim3(a.heads, num_entries, (a.N * a.P + 255) / 256),
                     dim3(256), 0, stream, a);
  hipLaunchKernelGGL((recurrence_kernel<NI, CPT, 8, false, false, kRecOutput>), grid,
                     dim3(kRecThreads), lds, stream, a);
}

template <int NI, int CPT, int SL>
static int launch_recurrence_cols(const RecurrenceArgs& a, int num_entries, bool delta, bool per_row,
                                  hipStream_t stream) {
  constexpr int LP = SL * (NI + 4), BC = kRecThreads / SL * CPT;
  const dim3 grid(a.heads, num_entries, (a.P + BC - 1) / BC);
  const dim3 block(kRecThreads);
  const int buf = (kRecStage * (2 * LP + (per_row ? LP : 1) + BC + 1) + 3) / 4 * 4;
  const size_t lds = (size_t)2 * buf * sizeof(float);
  const void* fn = delta && per_row ? (const void*)recurrence_kernel<NI, CPT, SL, true, true>
                   : delta          ? (const void*)recurrence_kernel<NI, CPT, SL, true, false>
                                    : (const void*)recurrence_kernel<NI, CPT, SL, false, false>;
  if (lds > 64 * 1024 &&
      hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return -1;
  if (delta && per_row)
    hipLaunchKernelGGL((recurrence_kernel<NI, CPT, SL, true, true>), grid, block, lds, stream, a);
  else if (delta)
    hipLaunchKernelGGL((recurrence_kernel<NI, CPT, SL, true, false>), grid, block, lds, stream, a);
  else
    hipLaunchKernelGGL((recurrence_kernel<NI, CPT, SL, false, false>), grid, block, lds, stream, a);
  return 0;
}

// `ni8`: rows a lane keeps when eight lanes share a column (a power of two from 2 to 32).
// Eight lanes and four columns a thread where the launch has workgroups enough (a step of many
// entries streams its states in wider rows); sixteen lanes and one column a thread where a few
// entries' long portions are walked.
template <int NI8>
static int launch_recurrence(const RecurrenceArgs& a, int num_entries, bool delta, bool per_row,
                             bool narrow, hipStream_t stream) {
  if (narrow)
    return launch_recurrence_cols<(NI8 >= 4 ? NI8 / 2 : 2), 1, 16>(a, num_entries, delta, per_row,
                                                                  stream);
  if constexpr (NI8 <= 16)
    return launch_recurrence_cols<NI8, 4, 8>(a, num_entries, delta, per_row, stream);
  else        // (four columns of 32 rows a thread do not fit the registers)
    return launch_recurrence_cols<NI8, 1, 8>(a, num_entries, delta, per_row, stream);
}

// x [T, ld] float32 holds q, k (kv_heads x N each) and v (heads x P) at the given columns
// (`silu`: their SiLU is taken as they are read).  `decay` [heads]: fixed decays, or null and
// `gates` [T, ldg] holds beta (heads; read by the delta rule only) and then the decays, one
// per head or (`per_row`) one per head and row of S.  out [T, heads*P].  `max_q_len`: the
// most tokens an entry brings (it chooses the launch's shape, never a result).
// `num_chunks` 0: every entry is walked whole.  Else (without the delta rule) `chunks`
// [num_chunks, 3] cuts every entry into runs of tokens (first, one past the last, entry), in
// order, `entry_chunks` [B + 1] says which are whose, and chunk_state [num_chunks, heads, N,
// P], chunk_decay [num_chunks, heads] are scratch.
extern "C" int ts_linear_recurrence(const float* x, int ld, int q_col, int k_col, int v_col,
                                    const float* decay, const float* gates, int ldg, float* state,
                                    float* out, const int* positions, const int* entry_of_token,
                                    const int* q_start, const int* slot_ids, int num_tokens,
                                    int num_entries, int max_q_len, int heads, int kv_heads,
                                    int N, int P, int silu, int delta, int per_row,
                                    const int* chunks, const int* entry_chunks, int num_chunks,
                                    float* chunk_state, float* chunk_decay, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || N <= 0 || P <= 0)
    TS_FAIL("linear_recurrence: bad sizes heads=%d kv_heads=%d dim=%d vdim=%d", heads, kv_heads, N, P);
  if (N > 256) TS_FAIL("linear_recurrence: %d key channels, at most 256 are built", N);
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
                   ld, q_col, k_col, v_col, ldg, heads, kv_heads, N, P, silu,
                   chunks, entry_chunks, chunk_state, chunk_decay};
  const int ni = (N + 7) / 8;
  if (num_chunks > 0) {
    if (delta) TS_FAIL("linear_recurrence: the delta rule is not linear in S and runs whole");
    if (!chunks || !entry_chunks || !chunk_state || !chunk_decay)
      TS_FAIL("linear_recurrence: chunked without its lists and scratch");
    if (ni > 16) TS_FAIL("linear_recurrence: chunks are built for up to 128 key channels");
    if (ni <= 2) launch_recurrence_chunked<2, 4>(a, num_entries, num_chunks, stream);
    else if (ni <= 4) launch_recurrence_chunked<4, 4>(a, num_entries, num_chunks, stream);
    else if (ni <= 8) launch_recurrence_chunked<8, 4>(a, num_entries, num_chunks, stream);
    else launch_recurrence_chunked<16, 4>(a, num_entries, num_chunks, stream);
    TS_CHECK_LAUNCH("linear_recurrence (chunked)");
    return 0;
  }
  const int64_t wide_groups = (int64_t)heads * num_entries * ((P + 63) / 64);
  const bool narrow = max_q_len >= 8 && wide_groups < 1024;
  int rc;
  if (ni <= 2) rc = launch_recurrence<2>(a, num_entries, delta, per_row, narrow, stream);
  else if (ni <= 4) rc = launch_recurrence<4>(a, num_entries, delta, per_row, narrow, stream);
  else if (ni <= 8) rc = launch_recurrence<8>(a, num_entries, delta, per_row, narrow, stream);
  else if (ni <= 16) rc = launch_recurrence<16>(a, num_entries, delta, per_row, narrow, stream);
  else rc = launch_recurrence<32>(a, num_entries, delta, per_row, narrow, stream);
  if (rc != 0) TS_FAIL("linear_recurrence: %d key channels need more LDS than the device gives", N);
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
