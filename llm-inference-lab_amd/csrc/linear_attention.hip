// Gated linear attention: a matrix-valued recurrent state per head,
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,
// with a decay a_t in (0, 1) per key channel.  The state [D, E] per head lives in float32 in
// a slot per request and is carried from step to step; everything here is float32.  gfx950.
//
// Three kernels: the decays from their low-rank projection; the scan over the tokens of every
// request of the step (prompts' portions and single decoded tokens alike); the output
// (norm over each head's values, gate, rounding to the compute dtype).
#include "common.h"

extern "C" const char* llmlab_last_error() { return g_llmlab_error; }

constexpr int SLICE = 16;      // key channels of the state that one thread keeps in registers

// ---------------------------------------------------------------------- decays
// a[r, c] = sigmoid(z)^(1 / tau), z = bias[c] + sum_j w2[c, j] * low[r, j]  (c over heads * D
// key channels, j over the rank of the projection).  sigmoid(z)^(1/tau) = exp(-softplus(-z) / tau),
// with softplus(u) = max(u, 0) + log1p(exp(-|u|)), so that neither end overflows.
__global__ __launch_bounds__(256) void gla_decay_kernel(const float* __restrict__ low, int ld, int rank,
                                                        const float* __restrict__ w2, const float* __restrict__ bias,
                                                        float inv_tau, float* __restrict__ decay, int channels) {
  const int r = blockIdx.x;
  const float* t = low + (size_t)r * ld;
  for (int c = threadIdx.x; c < channels; c += blockDim.x) {
    float z = bias ? bias[c] : 0.f;
    const float* w = w2 + (size_t)c * rank;
    for (int j = 0; j < rank; ++j) z = fmaf(w[j], t[j], z);
    const float u = -z;
    const float sp = fmaxf(u, 0.f) + log1pf(expf(-fabsf(u)));
    decay[(size_t)r * channels + c] = expf(-sp * inv_tau);
  }
}

extern "C" int llmlab_gla_decay(const float* low, int ld, int rows, int rank, const float* w2, const float* bias,
                                float tau, float* decay, int channels, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && rank > 0 && channels > 0 && ld >= rank && tau > 0.f,
                 "gla_decay: bad sizes rows=%d rank=%d channels=%d ld=%d tau=%g", rows, rank, channels, ld, (double)tau);
  if (rows == 0) return 0;
  hipLaunchKernelGGL(gla_decay_kernel, dim3(rows), dim3(256), 0, stream, low, ld, rank, w2, bias, 1.0f / tau, decay,
                     channels);
  LLMLAB_LAUNCH_CHECK("gla_decay");
  return 0;
}

// ------------------------------------------------------------------------ scan
// Thread (s, e) of a block keeps the SLICE rows s * SLICE .. of column e of one head's state in
// registers, walks a run of rows in order, and leaves its part of o_t in parts[row, h, s, e];
// the output kernel adds the parts of the slices.  Threads never talk to each other, so a
// token costs no barrier; the loads of a token do not depend on the state, so they run
// ahead of the sums.
//
// WHOLE: a block takes all the rows that request blockIdx.x brings to the step: the state
// comes from the request's slot and goes back there.  That is the kernel of decode steps
// and of short portions.
//
// Long portions are cut into chunks of `chunk` rows that run side by side, in three passes
// (the recurrence is linear in the state: S_end = P * S_start + L with P the product of the
// chunk's decays and L the state the chunk builds from zero):
//   LOCAL  per chunk: L and P, from a zero state, no outputs;
//   carry  per request, chunk after chunk: S_start[c], and the request's slot at the end;
//   FINISH per chunk: the rows again from S_start[c], now with outputs.
// All of it in float32; the result differs from the row-by-row recurrence by rounding only.
enum { SCAN_WHOLE = 0, SCAN_LOCAL = 1, SCAN_FINISH = 2 };

struct ScanArgs {
  const float* proj; int ld, off_q, off_k, off_v;
  const float* decay; float q_scale; int n_heads, D, E, cols, slices;
  float* state; const int* q_start; const int* req_rows; float* parts;
  int n_reqs, chunk; float* chunk_state; float* chunk_decay;      // [chunks, heads, D, E] and [chunks, heads, D]
};

// Which request and which rows the chunk `index` of the step covers (chunks are counted
// request after request); false if the step has fewer chunks.
__device__ __forceinline__ bool find_chunk(const ScanArgs& a, int index, int& first, int& last) {
  int before = 0;
  for (int b = 0; b < a.n_reqs; ++b) {
    const int lo = a.q_start[b], hi = a.q_start[b + 1];
    const int n = (hi - lo + a.chunk - 1) / a.chunk;
    if (index < before + n) {
      first = lo + (index - before) * a.chunk;
      last = first + a.chunk < hi ? first + a.chunk : hi;
      return true;
    }
    before += n;
  }
  return false;
}

template <int MODE, bool UNIFORM, int THREADS>
__global__ __launch_bounds__(THREADS) void gla_scan_kernel(ScanArgs a) {
  const int h = blockIdx.y;
  const int e = blockIdx.z * a.cols + (int)(threadIdx.x % a.cols);
  // UNIFORM: a wave lies within one slice (cols a multiple of 64), so the slice's decays,
  // keys and queries are the same for all its lanes and can come through the scalar unit
  const int s = UNIFORM ? __builtin_amdgcn_readfirstlane((int)(threadIdx.x / a.cols)) : (int)(threadIdx.x / a.cols);
  int first, last;
  if (MODE == SCAN_WHOLE) {
    first = a.q_start[blockIdx.x];
    last = a.q_start[blockIdx.x + 1];
  } else if (!find_chunk(a, blockIdx.x, first, last)) {
    return;
  }
  if (e >= a.E || s >= a.slices) return;
  const int D = a.D, E = a.E, d0 = s * SLICE;
  float S[SLICE], P[SLICE];
  float* st = MODE == SCAN_WHOLE ? a.state + (((size_t)a.req_rows[blockIdx.x] * a.n_heads + h) * D + d0) * E + e
                                 : a.chunk_state + (((size_t)blockIdx.x * a.n_heads + h) * D + d0) * E + e;
#pragma unroll
  for (int i = 0; i < SLICE; ++i) {
    S[i] = (MODE != SCAN_LOCAL && d0 + i < D) ? st[(size_t)i * E] : 0.f;
    P[i] = 1.f;
  }
  // A row's decays, keys, queries and value are asked for one row ahead, so that their way
  // from memory overlaps the sums of the row before; two sets of registers take turns, so
  // nothing is copied.
  const bool whole = d0 + SLICE <= D;
  struct Row {
    float a[SLICE], k[SLICE], q[SLICE], v;
  };
  auto fetch = [&](Row& r, int t) {
    const float* row = a.proj + (size_t)t * a.ld;
    const float* qp = row + a.off_q + h * D + d0;
    const float* kp = row + a.off_k + h * D + d0;
    const float* ap = a.decay + ((size_t)t * a.n_heads + h) * D + d0;
    r.v = row[a.off_v + h * E + e];
#pragma unroll
    for (int i = 0; i < SLICE; ++i) {
      const bool in = whole || d0 + i < D;
      r.a[i] = in ? ap[i] : 1.f;
      r.k[i] = in ? kp[i] : 0.f;
      if (MODE != SCAN_LOCAL) r.q[i] = in ? qp[i] : 0.f;
    }
  };
  auto take = [&](const Row& r, int t) {
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < SLICE; ++i) {
      S[i] = fmaf(r.a[i], S[i], r.k[i] * r.v);
      if (MODE == SCAN_LOCAL) P[i] *= r.a[i];
      else acc = fmaf(S[i], r.q[i], acc);
    }
    if (MODE != SCAN_LOCAL) a.parts[(((size_t)t * a.n_heads + h) * a.slices + s) * E + e] = acc * a.q_scale;
  };
  Row r0, r1;
  if (first < last) fetch(r0, first);
  for (int t = first; t < last; t += 2) {
    if (t + 1 < last) fetch(r1, t + 1);
    take(r0, t);
    if (t + 1 < last) {
      if (t + 2 < last) fetch(r0, t + 2);
      take(r1, t + 1);
    }
  }
  if (MODE == SCAN_FINISH) return;
#pragma unroll
  for (int i = 0; i < SLICE; ++i)
    if (d0 + i < D) st[(size_t)i * E] = S[i];
  if (MODE == SCAN_LOCAL && e == 0) {
    float* pd = a.chunk_decay + ((size_t)blockIdx.x * a.n_heads + h) * D + d0;
#pragma unroll
    for (int i = 0; i < SLICE; ++i)
      if (d0 + i < D) pd[i] = P[i];
  }
}

// One thread per element (h, d, e) of a request's state, chunk after chunk:
// chunk_state[c] <- the state before chunk c; the slot <- the state after the last chunk.
__global__ __launch_bounds__(256) void gla_carry_kernel(ScanArgs a) {
  const int b = blockIdx.y;
  const size_t per = (size_t)a.n_heads * a.D * a.E;
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= per) return;
  int before = 0;
  for (int r = 0; r < b; ++r) before += (a.q_start[r + 1] - a.q_start[r] + a.chunk - 1) / a.chunk;
  const int n = (a.q_start[b + 1] - a.q_start[b] + a.chunk - 1) / a.chunk;
  float* slot = a.state + (size_t)a.req_rows[b] * per + i;
  float S = *slot;
  const size_t hd = i / a.E;
  for (int c = before; c < before + n; ++c) {
    float* l = a.chunk_state + (size_t)c * per + i;
    const float built = *l;
    *l = S;
    S = fmaf(a.chunk_decay[(size_t)c * a.n_heads * a.D + hd], S, built);
  }
  *slot = S;
}

extern "C" int llmlab_gla_slices(int D) { return (D + SLICE - 1) / SLICE; }

// proj [rows, ld] float32 holds q at off_q (heads * D), k at off_k, v at off_v (heads * E);
// decay [rows, heads * D]; state [slots, heads, D, E]; parts [rows, heads, slices, E].
// chunk > 0: the three-pass form over chunks of so many rows; chunk_state then holds
// max_chunks * heads * D * E floats and chunk_decay max_chunks * heads * D, with max_chunks >=
// rows / chunk + n_reqs.
extern "C" int llmlab_gla_scan(const float* proj, int ld, int off_q, int off_k, int off_v, const float* decay,
                               float q_scale, int n_heads, int D, int E, float* state, const int* q_start,
                               const int* req_rows, int n_reqs, float* parts, int rows, int chunk,
                               float* chunk_state, float* chunk_decay, int max_chunks, hipStream_t stream) {
  LLMLAB_REQUIRE(n_reqs >= 0 && n_heads > 0 && D > 0 && E > 0, "gla_scan: bad sizes reqs=%d heads=%d D=%d E=%d", n_reqs,
                 n_heads, D, E);
  const int slices = (D + SLICE - 1) / SLICE;
  int cols = E < 64 ? E : 64;
  while (cols > 1 && slices * cols > 1024) cols /= 2;
  LLMLAB_REQUIRE(slices * cols <= 1024, "gla_scan: %d key channels per head are more than a block holds", D);
  LLMLAB_REQUIRE(n_heads <= 65535 && (E + cols - 1) / cols <= 65535 && n_reqs <= 65535,
                 "gla_scan: too many heads, columns or requests");
  if (n_reqs == 0) return 0;
  ScanArgs a{proj, ld, off_q, off_k, off_v, decay, q_scale, n_heads, D, E, cols, slices, state, q_start, req_rows, parts,
             n_reqs, chunk, chunk_state, chunk_decay};
  const bool uniform = cols == 64;
  dim3 block(slices * cols);
  const unsigned slabs = (E + cols - 1) / cols;
  // (blocks of up to 256 threads, heads of up to 64 key channels, are compiled with the
  // registers that leaves them: the rows fetched ahead stay in registers then)
  const bool small = slices * cols <= 256;
#define LLMLAB_SCAN(MODE, GRIDX)                                                                                  \
  do {                                                                                                            \
    const dim3 grid_(GRIDX, n_heads, slabs);                                                                      \
    if (uniform && small) hipLaunchKernelGGL((gla_scan_kernel<MODE, true, 256>), grid_, block, 0, stream, a);     \
    else if (uniform) hipLaunchKernelGGL((gla_scan_kernel<MODE, true, 1024>), grid_, block, 0, stream, a);        \
    else if (small) hipLaunchKernelGGL((gla_scan_kernel<MODE, false, 256>), grid_, block, 0, stream, a);          \
    else hipLaunchKernelGGL((gla_scan_kernel<MODE, false, 1024>), grid_, block, 0, stream, a);                    \
  } while (0)
  if (chunk <= 0) {
    LLMLAB_SCAN(SCAN_WHOLE, n_reqs);
  } else {
    const int chunks = rows / chunk + n_reqs;
    LLMLAB_REQUIRE(chunk_state && chunk_decay && max_chunks >= chunks,
                   "gla_scan: %d rows of %d requests in chunks of %d need room for %d chunks, got %d", rows, n_reqs,
                   chunk, chunks, max_chunks);
    LLMLAB_SCAN(SCAN_LOCAL, chunks);
    const size_t per = (size_t)n_heads * D * E;
    hipLaunchKernelGGL(gla_carry_kernel, dim3((unsigned)((per + 255) / 256), n_reqs), dim3(256), 0, stream, a);
    LLMLAB_SCAN(SCAN_FINISH, chunks);
  }
#undef LLMLAB_SCAN
  LLMLAB_LAUNCH_CHECK("gla_scan");
  return 0;
}

// ---------------------------------------------------------------------- output
// Block (row, head): o = sum over slices of parts; y = o / sqrt(mean(o^2) + eps) * w[e]
// (the weight has one entry per value channel, the same for every head; w_per_head: one per
// head and channel, w[h * E + e]); out = T(y * silu(gate)), silu(g) = g / (1 + exp(-g))
// (gate_kind 1: y * sigmoid(gate)); gate [rows, ld] float32 at column off_g.
template <typename T>
__global__ __launch_bounds__(1024) void gla_output_kernel(const float* __restrict__ parts, int slices, int n_heads, int E,
                                                          const float* __restrict__ w, float eps,
                                                          const float* __restrict__ proj, int ld, int off_g,
                                                          T* __restrict__ out, int w_per_head, int gate_kind) {
  __shared__ float red[17];
  const int r = blockIdx.x, h = blockIdx.y, e = threadIdx.x;
  float o = 0.f;
  if (e < E) {
    const float* p = parts + (((size_t)r * n_heads + h) * slices) * E + e;
    for (int s = 0; s < slices; ++s) o += p[(size_t)s * E];
  }
  const float ms = block_sum(o * o, red) / (float)E;
  if (e < E) {
    const float g = proj[(size_t)r * ld + off_g + h * E + e];
    const float y = o * (1.0f / sqrtf(ms + eps)) * w[w_per_head ? h * E + e : e];
    const float sg = 1.0f / (1.0f + expf(-g));
    out[((size_t)r * n_heads + h) * E + e] = from_float<T>(y * (gate_kind == 1 ? sg : g * sg));
  }
}

// slices > 0: that many pieces per output (0: as the gated scan leaves them, one per SLICE key channels)
extern "C" int llmlab_gla_output(const float* parts, int rows, int n_heads, int D, int E, const float* w, float eps,
                                 const float* proj, int ld, int off_g, void* out, int dtype, int slices_given,
                                 int w_per_head, int gate_kind, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && n_heads > 0 && n_heads <= 65535 && E > 0 && E <= 1024,
                 "gla_output: bad sizes rows=%d heads=%d E=%d", rows, n_heads, E);
  LLMLAB_REQUIRE(gate_kind == 0 || gate_kind == 1, "gla_output: unknown gate %d", gate_kind);
  if (rows == 0) return 0;
  const int slices = slices_given > 0 ? slices_given : (D + SLICE - 1) / SLICE;
  dim3 grid(rows, n_heads), block((E + 63) / 64 * 64);
  if (dtype == DT_BF16)
    hipLaunchKernelGGL(gla_output_kernel<bf16_t>, grid, block, 0, stream, parts, slices, n_heads, E, w, eps, proj, ld,
                       off_g, (bf16_t*)out, w_per_head, gate_kind);
  else
    hipLaunchKernelGGL(gla_output_kernel<float>, grid, block, 0, stream, parts, slices, n_heads, E, w, eps, proj, ld,
                       off_g, (float*)out, w_per_head, gate_kind);
  LLMLAB_LAUNCH_CHECK("gla_output");
  return 0;
}


// ================================================================== generalised delta rule
// A matrix-valued state per head whose transition is a decay per key channel less a rank-one
// removal along the unit key, before the new key/value pair is written:
//   u_t = k_t / sqrt(|k_t|^2 + key_eps)
//   S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T        (both terms read S_(t-1))
//   o_t = S_t^T r_t
// with w_t (decay) and a_t (removal rate) in (0, 1) per head and key channel.  State [D, E]
// per head, float32, one slot per request; everything here is float32.
//
// delta_gates: w = exp(-decay_scale * sigmoid(w0 + W2 tanh(low))) from the low-rank projection
// `low` (rank numbers a row), a = sigmoid(a_in + a_bias).
__global__ __launch_bounds__(256) void delta_gates_kernel(const float* __restrict__ proj, int ld, int off_low, int rank,
                                                          int off_a, const float* __restrict__ w2,
                                                          const float* __restrict__ w0, const float* __restrict__ a_bias,
                                                          float decay_scale, float* __restrict__ decay,
                                                          float* __restrict__ rate, int channels) {
  extern __shared__ float s_low[];       // tanh of the row's low-rank numbers
  const int r = blockIdx.x;
  const float* t = proj + (size_t)r * ld;
  for (int j = threadIdx.x; j < rank; j += blockDim.x) s_low[j] = tanhf(t[off_low + j]);
  __syncthreads();
  for (int c = threadIdx.x; c < channels; c += blockDim.x) {
    float z = w0 ? w0[c] : 0.f;
    const float* w = w2 + (size_t)c * rank;
    for (int j = 0; j < rank; ++j) z = fmaf(w[j], s_low[j], z);
    decay[(size_t)r * channels + c] = expf(-decay_scale / (1.0f + expf(-z)));
    const float za = t[off_a + c] + (a_bias ? a_bias[c] : 0.f);
    rate[(size_t)r * channels + c] = 1.0f / (1.0f + expf(-za));
  }
}

extern "C" int llmlab_delta_gates(const float* proj, int ld, int rows, int off_low, int rank, int off_a, const float* w2,
                                  const float* w0, const float* a_bias, float decay_scale, float* decay, float* rate,
                                  int channels, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && rank > 0 && rank <= 8192 && channels > 0 && off_low >= 0 && off_a >= 0 &&
                 ld >= off_low + rank && ld >= off_a + channels,
                 "delta_gates: bad sizes rows=%d rank=%d channels=%d ld=%d", rows, rank, channels, ld);
  if (rows == 0) return 0;
  hipLaunchKernelGGL(delta_gates_kernel, dim3(rows), dim3(256), rank * sizeof(float), stream, proj, ld, off_low, rank,
                     off_a, w2, w0, a_bias, decay_scale, decay, rate, channels);
  LLMLAB_LAUNCH_CHECK("delta_gates");
  return 0;
}

// delta_scan: thread e of block (request, head) keeps column e of the head's state (DK >= D
// numbers) in registers and walks the request's rows of the step in order; the row's key,
// receptance, decay and rate are the same for every thread of the block (uniform loads), its
// value is one number a thread.  No thread talks to another, so a token costs no barrier.
// Rows [row_begin, row_end) of the request: the state comes from `s_in` and goes to `s_out`
// (both [D, E] of this head; s_in null: zero).
template <int DK>
__device__ __forceinline__ void delta_walk(const float* __restrict__ proj, int ld, int off_r, int off_k, int off_v,
                                           const float* __restrict__ decay, const float* __restrict__ rate, int n_heads,
                                           int h, int D, int E, float key_eps, int row_begin, int row_end,
                                           const float* __restrict__ s_in, float* __restrict__ s_out,
                                           float* __restrict__ out, int e) {
  float S[DK];
#pragma unroll
  for (int d = 0; d < DK; ++d) S[d] = (s_in && d < D && e < E) ? s_in[(size_t)d * E + e] : 0.f;
  const int ec = e < E ? e : E - 1;
  for (int t = row_begin; t < row_end; ++t) {
    const float* row = proj + (size_t)t * ld;
    const float* kk = row + off_k + h * D;
    const float* rr = row + off_r + h * D;
    const float* ww = decay + ((size_t)t * n_heads + h) * D;
    const float* aa = rate + ((size_t)t * n_heads + h) * D;
    const float v = row[off_v + h * E + ec];
    float k2 = 0.f;
#pragma unroll
    for (int d = 0; d < DK; ++d)
      if (d < D) k2 = fmaf(kk[d], kk[d], k2);
    const float inv = 1.0f / sqrtf(k2 + key_eps);
    float dot = 0.f;
#pragma unroll
    for (int d = 0; d < DK; ++d)
      if (d < D) dot = fmaf(kk[d] * inv, S[d], dot);
    float o = 0.f;
#pragma unroll
    for (int d = 0; d < DK; ++d)
      if (d < D) {
        const float k = kk[d];
        S[d] = fmaf(ww[d], S[d], fmaf(-(aa[d] * (k * inv)), dot, k * v));
        o = fmaf(S[d], rr[d], o);
      }
    if (e < E) out[((size_t)t * n_heads + h) * E + e] = o;
  }
  if (e < E) {
#pragma unroll
    for (int d = 0; d < DK; ++d)
      if (d < D) s_out[(size_t)d * E + e] = S[d];
  }
}

template <int DK>
__global__ __launch_bounds__(256) void delta_scan_kernel(const float* __restrict__ proj, int ld, int off_r, int off_k,
                                                         int off_v, const float* __restrict__ decay,
                                                         const float* __restrict__ rate, int n_heads, int D, int E,
                                                         float key_eps, float* __restrict__ state,
                                                         const int* __restrict__ q_start, const int* __restrict__ req_rows,
                                                         float* __restrict__ out) {
  const int b = blockIdx.x, h = blockIdx.y;
  const int e = blockIdx.z * blockDim.x + threadIdx.x;
  float* st = state + ((size_t)req_rows[b] * n_heads + h) * D * E;
  delta_walk<DK>(proj, ld, off_r, off_k, off_v, decay, rate, n_heads, h, D, E, key_eps, q_start[b], q_start[b + 1], st, st,
                 out, e);
}

extern "C" int llmlab_delta_scan(const float* proj, int ld, int off_r, int off_k, int off_v, const float* decay,
                                 const float* rate, int n_heads, int D, int E, float key_eps, float* state,
                                 const int* q_start, const int* req_rows, int n_reqs, float* out, int rows,
                                 hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && n_reqs >= 0 && n_heads > 0 && n_heads <= 65535 && D > 0 && D <= 256 && E > 0 && E <= 16384,
                 "delta_scan: bad sizes rows=%d requests=%d heads=%d D=%d E=%d (keys up to 256 wide)", rows, n_reqs,
                 n_heads, D, E);
  LLMLAB_REQUIRE(off_r >= 0 && off_k >= 0 && off_v >= 0 && ld >= off_r + n_heads * D && ld >= off_k + n_heads * D &&
                 ld >= off_v + n_heads * E, "delta_scan: rows of %d numbers do not hold the projections", ld);
  if (rows == 0 || n_reqs == 0) return 0;
  const int threads = E <= 64 ? 64 : (E <= 128 ? 128 : 256);
  dim3 grid(n_reqs, n_heads, (E + threads - 1) / threads), block(threads);
#define LLMLAB_DELTA(DKV)                                                                                             \
  hipLaunchKernelGGL(delta_scan_kernel<DKV>, grid, block, 0, stream, proj, ld, off_r, off_k, off_v, decay, rate, n_heads, \
                     D, E, key_eps, state, q_start, req_rows, out)
  if (D <= 16) LLMLAB_DELTA(16);
  else if (D <= 32) LLMLAB_DELTA(32);
  else if (D <= 64) LLMLAB_DELTA(64);
  else if (D <= 128) LLMLAB_DELTA(128);
  else LLMLAB_DELTA(256);
#undef LLMLAB_DELTA
  LLMLAB_LAUNCH_CHECK("delta_scan");
  return 0;
}
