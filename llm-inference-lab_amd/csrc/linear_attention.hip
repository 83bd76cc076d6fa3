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
                                                          T* __restrict__ out, int w_per_head, int gate_kind,
                                                          int count) {
  __shared__ float red[17];
  const int r = blockIdx.x, h = blockIdx.y, e = threadIdx.x;
  float o = 0.f;
  if (e < E) {
    const float* p = parts + (((size_t)r * n_heads + h) * slices) * E + e;
    for (int s = 0; s < slices; ++s) o += p[(size_t)s * E];
  }
  const float ms = block_sum(o * o, red) / (float)count;      // (count < E: the channels behind it are zeros)
  if (e < E) {
    const float g = proj[(size_t)r * ld + off_g + h * E + e];
    const float y = o * (1.0f / sqrtf(ms + eps)) * w[w_per_head ? h * E + e : e];
    const float sg = 1.0f / (1.0f + expf(-g));
    out[((size_t)r * n_heads + h) * E + e] = from_float<T>(y * (gate_kind == 1 ? sg : g * sg));
  }
}

// slices > 0: that many pieces per output (0: as the gated scan leaves them, one per SLICE key channels);
// norm_count > 0: the mean of the squares is taken over so many channels (the others are zeros)
extern "C" int llmlab_gla_output(const float* parts, int rows, int n_heads, int D, int E, const float* w, float eps,
                                 const float* proj, int ld, int off_g, void* out, int dtype, int slices_given,
                                 int w_per_head, int gate_kind, int norm_count, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && n_heads > 0 && n_heads <= 65535 && E > 0 && E <= 1024,
                 "gla_output: bad sizes rows=%d heads=%d E=%d", rows, n_heads, E);
  LLMLAB_REQUIRE(gate_kind == 0 || gate_kind == 1, "gla_output: unknown gate %d", gate_kind);
  LLMLAB_REQUIRE(norm_count >= 0 && norm_count <= E, "gla_output: a mean over %d of %d channels", norm_count, E);
  const int count = norm_count > 0 ? norm_count : E;
  if (rows == 0) return 0;
  const int slices = slices_given > 0 ? slices_given : (D + SLICE - 1) / SLICE;
  dim3 grid(rows, n_heads), block((E + 63) / 64 * 64);
  if (dtype == DT_BF16)
    hipLaunchKernelGGL(gla_output_kernel<bf16_t>, grid, block, 0, stream, parts, slices, n_heads, E, w, eps, proj, ld,
                       off_g, (bf16_t*)out, w_per_head, gate_kind, count);
  else
    hipLaunchKernelGGL(gla_output_kernel<float>, grid, block, 0, stream, parts, slices, n_heads, E, w, eps, proj, ld,
                       off_g, (float*)out, w_per_head, gate_kind, count);
  LLMLAB_LAUNCH_CHECK("gla_output");
  return 0;
}


// ================================================================== generalised delta rule
// A matrix-valued state per head whose transition is a decay per key channel less a rank-one
// removal along the unit key, before the new key/value pair is written:
//   u_t = k_t / sqrt(|k_t|^2 + key_eps)
//   S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T        (decay and removal act on S_(t-1))
//   o_t = S_t^T r_t
// with w_t (decay) and a_t (removal rate) in (0, 1) per head and key channel.  State [D, E]
// per head, float32, one slot per request; everything here is float32.
//
// delta_gates, one block a row: w = exp(-decay_scale * sigmoid(w0 + W2 tanh(low))) from the
// low-rank projection `low` (rank numbers a row), a = sigmoid(a_in + a_bias), and what every
// column of the state needs of the row's key: the unit key u and the removal a * u.
constexpr int GATES_MAX_HEADS = 1024;
__global__ __launch_bounds__(256) void delta_gates_kernel(const float* __restrict__ proj, int ld, int off_low, int rank,
                                                          int off_a, int off_k, const float* __restrict__ w2,
                                                          const float* __restrict__ w0, const float* __restrict__ a_bias,
                                                          float decay_scale, float key_eps, float* __restrict__ decay,
                                                          float* __restrict__ unit, float* __restrict__ removal,
                                                          int n_heads, int D) {
  extern __shared__ float s_low[];       // tanh of the row's low-rank numbers, then 1 / |k| of every head
  float* s_inv = s_low + rank;
  const int r = blockIdx.x, channels = n_heads * D;
  const float* t = proj + (size_t)r * ld;
  for (int j = threadIdx.x; j < rank; j += blockDim.x) s_low[j] = tanhf(t[off_low + j]);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  for (int h = wave; h < n_heads; h += waves) {          // a wave a head
    float k2 = 0.f;
    for (int d = lane; d < D; d += 64) {
      const float k = t[off_k + h * D + d];
      k2 = fmaf(k, k, k2);
    }
    k2 = wave_sum(k2);
    if (lane == 0) s_inv[h] = 1.0f / sqrtf(k2 + key_eps);
  }
  __syncthreads();
  for (int c = threadIdx.x; c < channels; c += blockDim.x) {
    float z = w0 ? w0[c] : 0.f;
    const float* w = w2 + (size_t)c * rank;
    const float za = t[off_a + c] + (a_bias ? a_bias[c] : 0.f);
    const float u = t[off_k + c] * s_inv[c / D];
    if ((rank & 3) == 0) {                       // (a row of the second factor 16 bytes a load, all on their way together)
      for (int j = 0; j < rank; j += 4) {
        const floatx4 w4 = *(const floatx4*)(w + j);
        z = fmaf(w4[0], s_low[j], z);
        z = fmaf(w4[1], s_low[j + 1], z);
        z = fmaf(w4[2], s_low[j + 2], z);
        z = fmaf(w4[3], s_low[j + 3], z);
      }
    } else {
      for (int j = 0; j < rank; ++j) z = fmaf(w[j], s_low[j], z);
    }
    decay[(size_t)r * channels + c] = expf(-decay_scale / (1.0f + expf(-z)));
    unit[(size_t)r * channels + c] = u;
    removal[(size_t)r * channels + c] = u / (1.0f + expf(-za));
  }
}

extern "C" int llmlab_delta_gates(const float* proj, int ld, int rows, int off_low, int rank, int off_a, int off_k,
                                  const float* w2, const float* w0, const float* a_bias, float decay_scale,
                                  float key_eps, float* decay, float* unit, float* removal, int n_heads, int D,
                                  hipStream_t stream) {
  const int channels = n_heads * D;
  LLMLAB_REQUIRE(rows >= 0 && rank > 0 && rank <= 8192 && n_heads > 0 && n_heads <= GATES_MAX_HEADS && D > 0 &&
                 off_low >= 0 && off_a >= 0 && off_k >= 0 && ld >= off_low + rank && ld >= off_a + channels &&
                 ld >= off_k + channels,
                 "delta_gates: bad sizes rows=%d rank=%d heads=%d D=%d ld=%d", rows, rank, n_heads, D, ld);
  if (rows == 0) return 0;
  hipLaunchKernelGGL(delta_gates_kernel, dim3(rows), dim3(256), (rank + n_heads) * sizeof(float), stream, proj, ld,
                     off_low, rank, off_a, off_k, w2, w0, a_bias, decay_scale, key_eps, decay, unit, removal, n_heads, D);
  LLMLAB_LAUNCH_CHECK("delta_gates");
  return 0;
}

// delta_scan.  A quad of lanes keeps ONE column of a head's state in registers, a quarter of its
// DK >= D numbers each (the two sums over a column meet across the quad), and walks rows in order; the row's decay, unit key, removal, key and receptance are the same for
// every column: the block brings them into LDS a group of rows ahead (two buffers take turns, one
// barrier and one wait for memory a group), its value is one number a thread.  Per row and column: the dot product of the unit
// key with the column, the update, the dot product with the receptance.
//
// WHOLE: a block takes all the rows that a request brings to the step, for one head and 64
// columns: state from the request's slot and back.  Decode steps and short portions.
//
// Long portions are cut into chunks that run side by side, in three passes.  The recurrence is
// linear in the state, S_end = T S_start + L, with T (D x D) the product of the chunk's
// transitions diag(w) - (a * u) u^T and L the state the chunk builds from zero.  A column of T is
// what the recurrence without values makes of a unit vector, so:
//   LOCAL  per chunk: the E columns of L from zero and the D columns of T from the identity, no outputs;
//   carry  per request, chunk after chunk: S_start[c + 1] = T_c S_start[c] + L_c; the slot at the end;
//   FINISH per chunk: the rows again from S_start[c], now with outputs.
enum { DELTA_WHOLE = 0, DELTA_LOCAL = 1, DELTA_FINISH = 2 };

struct DeltaArgs {
  const float* proj; int ld, off_r, off_k, off_v;
  const float* decay; const float* unit; const float* removal;      // [rows, heads * D]
  int n_heads, D, E;
  float* state; const int* q_start; const int* req_rows; float* out;      // out [rows, heads, E]
  int n_reqs, chunk; float* chunk_state; float* chunk_trans;      // [chunks, heads, D, E] and [chunks, heads, D, D]
};

__device__ __forceinline__ bool delta_find_chunk(const DeltaArgs& a, int index, int& first, int& last) {
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

// the sum of a number over the four lanes of a quad (lanes 4 n .. 4 n + 3), in every one of them
__device__ __forceinline__ float quad_sum(float x) {
  x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0xB1, 0xF, 0xF, true));      // lanes 1, 0, 3, 2
  x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x4E, 0xF, 0xF, true));      // lanes 2, 3, 0, 1
  return x;
}

template <int DK, int MODE>
__global__ __launch_bounds__(256) void delta_scan_kernel(DeltaArgs a) {
  constexpr int VECS = MODE == DELTA_LOCAL ? 4 : 5;      // decay, unit key, removal, key (, receptance)
  constexpr int DQ = DK / 4;                              // rows of a column that one lane of its quad keeps
  constexpr int PER = (VECS * DK + 255) / 256;            // numbers of a row that a thread brings
  constexpr int G = DK <= 64 ? 8 : (DK <= 128 ? 4 : 2);   // rows that travel together (one wait for memory per G rows)
  __shared__ __attribute__((aligned(16))) float tok[2][G][VECS][DK];
  const int h = blockIdx.y, D = a.D, E = a.E;
  const int q = threadIdx.x & 3, d0 = q * DQ;
  const int col = blockIdx.z * 64 + (int)(threadIdx.x >> 2);
  const int cols = MODE == DELTA_LOCAL ? E + D : E;
  int first, last;
  if (MODE == DELTA_WHOLE) {
    first = a.q_start[blockIdx.x];
    last = a.q_start[blockIdx.x + 1];
  } else if (!delta_find_chunk(a, blockIdx.x, first, last)) {
    return;
  }
  const bool live = col < cols;
  const bool is_value = col < E;                          // (LOCAL: the others are columns of the transition)
  const int e = is_value ? col : E - 1;
  float S[DQ];
  const float* s_in = MODE == DELTA_WHOLE ? a.state + ((size_t)a.req_rows[blockIdx.x] * a.n_heads + h) * D * E
                      : MODE == DELTA_FINISH ? a.chunk_state + ((size_t)blockIdx.x * a.n_heads + h) * D * E : nullptr;
#pragma unroll
  for (int i = 0; i < DQ; ++i) {
    const int d = d0 + i;
    if (MODE == DELTA_LOCAL) S[i] = (live && !is_value && d == col - E) ? 1.f : 0.f;
    else S[i] = (live && d < D) ? s_in[(size_t)d * E + e] : 0.f;
  }
  // the numbers of a row that this thread brings: number i of vector i / D, for i = tid, tid + 256, ...
  const int total = VECS * D;
  float pre[G][PER], v_pre[G], v_now[G];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      if (g > 0 && t0 + g >= last) break;                          // (a decode step brings one row)
      const int t = t0 + g;
      const float* row = a.proj + (size_t)t * a.ld;
      const size_t at = ((size_t)t * a.n_heads + h) * D;
      v_pre[g] = is_value ? row[a.off_v + h * E + e] : 0.f;
#pragma unroll
      for (int n = 0; n < PER; ++n) {
        const int i = threadIdx.x + n * 256;
        float x = 0.f;
        if (i < total) {
          const int vec = i / D, d = i - vec * D;
          x = vec == 0 ? a.decay[at + d] : vec == 1 ? a.unit[at + d] : vec == 2 ? a.removal[at + d]
              : vec == 3 ? row[a.off_k + h * D + d] : row[a.off_r + h * D + d];
        }
        pre[g][n] = x;
      }
    }
  };
  auto stash = [&](int buf, int t0) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      if (g > 0 && t0 + g >= last) break;
#pragma unroll
      for (int n = 0; n < PER; ++n) {
        const int i = threadIdx.x + n * 256;
        if (i < total) {
          const int vec = i / D, d = i - vec * D;
          tok[buf][g][vec][d] = pre[g][n];
        }
      }
    }
  };
  // (vectors shorter than DK: the rest stays zero, so the sums over DK numbers need no bound)
  if (D < DK)
    for (int i = threadIdx.x; i < 2 * G * VECS * DK; i += 256) (&tok[0][0][0][0])[i] = 0.f;
  __syncthreads();
  if (first < last) {
    fetch(first);
    stash(0, first);
  }
  __syncthreads();
  for (int t0 = first, buf = 0; t0 < last; t0 += G, buf ^= 1) {
#pragma unroll
    for (int g = 0; g < G; ++g) v_now[g] = v_pre[g];
    const bool more = t0 + G < last;
    if (more) fetch(t0 + G);
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const int t = t0 + g;
      if (t < last) {
        const float v = v_now[g];
        const float* w_ = &tok[buf][g][0][d0];
        const float* u_ = &tok[buf][g][1][d0];
        const float* au_ = &tok[buf][g][2][d0];
        const float* k_ = &tok[buf][g][3][d0];
        // (sums side by side, so that no sum waits for the one before it)
        float dots[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < DQ; ++i) dots[i & 3] = fmaf(u_[i], S[i], dots[i & 3]);
        const float dot = quad_sum((dots[0] + dots[1]) + (dots[2] + dots[3]));
        float os[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < DQ; ++i) {
          S[i] = fmaf(w_[i], S[i], fmaf(-au_[i], dot, k_[i] * v));
          if (MODE != DELTA_LOCAL) os[i & 3] = fmaf(S[i], tok[buf][g][VECS - 1][d0 + i], os[i & 3]);
        }
        if (MODE != DELTA_LOCAL) {
          const float o = quad_sum((os[0] + os[1]) + (os[2] + os[3]));
          if (live && q == 0) a.out[((size_t)t * a.n_heads + h) * E + e] = o;
        }
      }
    }
    if (more) stash(buf ^ 1, t0 + G);
    __syncthreads();
  }
  if (MODE == DELTA_FINISH || !live) return;
  float* dst;
  size_t stride;
  if (MODE == DELTA_WHOLE) {
    dst = a.state + ((size_t)a.req_rows[blockIdx.x] * a.n_heads + h) * D * E + e;
    stride = E;
  } else if (is_value) {
    dst = a.chunk_state + ((size_t)blockIdx.x * a.n_heads + h) * D * E + e;
    stride = E;
  } else {
    dst = a.chunk_trans + ((size_t)blockIdx.x * a.n_heads + h) * D * D + (col - E);
    stride = D;
  }
#pragma unroll
  for (int i = 0; i < DQ; ++i)
    if (d0 + i < D) dst[(size_t)(d0 + i) * stride] = S[i];
}

// carry: block (request, head, slab of 16 columns), CARRY_GROUPS waves; wave g computes the rows
// g, g + CARRY_GROUPS, ... of T_c S + L_c for the slab's columns: a column a quad of lanes, each lane
// a quarter of the sum over the old rows.  The slab of the state and the chunk's transition lie in
// LDS (a wave brings its own rows of the transition, the next chunk's while this chunk's sums are
// taken).  chunk_state[c] <- the state before chunk c.
constexpr int CARRY_GROUPS = 8, CARRY_COLS = 16;
template <int DK>
__global__ __launch_bounds__(64 * CARRY_GROUPS) void delta_carry_kernel(DeltaArgs a) {
  constexpr int ROWS = (DK + CARRY_GROUPS - 1) / CARRY_GROUPS, M = (DK + 63) / 64, DQ = DK / 4;
  __shared__ __attribute__((aligned(16))) float s_tr[ROWS * CARRY_GROUPS][DK + 4];
  __shared__ float s_col[DK][CARRY_COLS + 1];
  const int b = blockIdx.x, h = blockIdx.y, D = a.D, E = a.E;
  const int lane = threadIdx.x & 63, g = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int q = lane & 3, c16 = lane >> 2, j0 = q * DQ;
  const int e = blockIdx.z * CARRY_COLS + c16;
  const bool live = e < E;
  const int ec = live ? e : E - 1;
  int before = 0;
  for (int r = 0; r < b; ++r) before += (a.q_start[r + 1] - a.q_start[r] + a.chunk - 1) / a.chunk;
  const int n = (a.q_start[b + 1] - a.q_start[b] + a.chunk - 1) / a.chunk;
  float* slot = a.state + ((size_t)a.req_rows[b] * a.n_heads + h) * D * E;
  for (int i = threadIdx.x; i < DK * CARRY_COLS; i += blockDim.x) {
    const int d = i / CARRY_COLS, c = i % CARRY_COLS;
    const int ee = blockIdx.z * CARRY_COLS + c;
    s_col[d][c] = (d < D && ee < E) ? slot[(size_t)d * E + ee] : 0.f;
  }
  // this wave's rows of a chunk's transition (64 entries of a row a register) and of its built state
  float tr[ROWS][M], built[ROWS];
  auto fetch = [&](int c) {
    const float* lp = a.chunk_state + ((size_t)c * a.n_heads + h) * D * E;
    const float* tp = a.chunk_trans + ((size_t)c * a.n_heads + h) * D * D;
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      const int d = g + CARRY_GROUPS * i;
      built[i] = d < D ? lp[(size_t)d * E + ec] : 0.f;
#pragma unroll
      for (int m = 0; m < M; ++m) tr[i][m] = (d < D && 64 * m + lane < D) ? tp[(size_t)d * D + 64 * m + lane] : 0.f;
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < ROWS; ++i)
#pragma unroll
      for (int m = 0; m < M; ++m)
        if (64 * m + lane < DK) s_tr[g + CARRY_GROUPS * i][64 * m + lane] = tr[i][m];
  };
  if (n > 0) {
    fetch(before);
    stash();
  }
  __syncthreads();
  for (int c = before; c < before + n; ++c) {
    float acc[ROWS];
#pragma unroll
    for (int i = 0; i < ROWS; ++i) acc[i] = q == 0 ? built[i] : 0.f;
    if (c + 1 < before + n) fetch(c + 1);                          // (on its way while the sums are taken)
    float* l = a.chunk_state + ((size_t)c * a.n_heads + h) * D * E;
#pragma unroll
    for (int jj = 0; jj < DQ; ++jj) {
      const float x = s_col[j0 + jj][c16];
#pragma unroll
      for (int i = 0; i < ROWS; ++i) acc[i] = fmaf(s_tr[g + CARRY_GROUPS * i][j0 + jj], x, acc[i]);
    }
#pragma unroll
    for (int i = 0; i < ROWS; ++i) acc[i] = quad_sum(acc[i]);
    if (live && q == 0) {                                          // the state before this chunk, in the chunk's place
#pragma unroll
      for (int i = 0; i < ROWS; ++i) {
        const int d = g + CARRY_GROUPS * i;
        if (d < D) l[(size_t)d * E + e] = s_col[d][c16];
      }
    }
    __syncthreads();                                               // (every wave has read the old columns and the transition)
    if (q == 0) {
#pragma unroll
      for (int i = 0; i < ROWS; ++i) {
        const int d = g + CARRY_GROUPS * i;
        if (d < DK) s_col[d][c16] = acc[i];
      }
    }
    if (c + 1 < before + n) stash();
    __syncthreads();
  }
  if (live && q == 0)
    for (int d = g; d < D; d += CARRY_GROUPS) slot[(size_t)d * E + e] = s_col[d][c16];
}

// proj [rows, ld] float32 holds r at off_r (heads * D), k at off_k, v at off_v (heads * E); decay,
// unit and removal [rows, heads * D] (delta_gates); state [slots, heads, D, E]; out [rows, heads, E].
// chunk > 0: the three-pass form over chunks of so many rows; chunk_state then holds max_chunks *
// heads * D * E floats and chunk_trans max_chunks * heads * D * D, max_chunks >= rows / chunk + n_reqs.
extern "C" int llmlab_delta_scan(const float* proj, int ld, int off_r, int off_k, int off_v, const float* decay,
                                 const float* unit, const float* removal, int n_heads, int D, int E, float* state,
                                 const int* q_start, const int* req_rows, int n_reqs, float* out, int rows, int chunk,
                                 float* chunk_state, float* chunk_trans, int max_chunks, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && n_reqs >= 0 && n_reqs <= 65535 && n_heads > 0 && n_heads <= 65535 && D > 0 && D <= 256 &&
                 E > 0 && E <= 16384,
                 "delta_scan: bad sizes rows=%d requests=%d heads=%d D=%d E=%d (keys up to 256 wide)", rows, n_reqs,
                 n_heads, D, E);
  LLMLAB_REQUIRE(off_r >= 0 && off_k >= 0 && off_v >= 0 && ld >= off_r + n_heads * D && ld >= off_k + n_heads * D &&
                 ld >= off_v + n_heads * E, "delta_scan: rows of %d numbers do not hold the projections", ld);
  if (rows == 0 || n_reqs == 0) return 0;
  DeltaArgs a{proj, ld, off_r, off_k, off_v, decay, unit, removal, n_heads, D, E, state, q_start, req_rows, out,
              n_reqs, chunk, chunk_state, chunk_trans};
#define LLMLAB_DELTA(DKV, MODE, GRIDX, COLS) \
  hipLaunchKernelGGL((delta_scan_kernel<DKV, MODE>), dim3(GRIDX, n_heads, ((COLS) + 63) / 64), dim3(256), 0, stream, a)
#define LLMLAB_DELTA_ANY(MODE, GRIDX, COLS)                   \
  do {                                                        \
    if (D <= 16) LLMLAB_DELTA(16, MODE, GRIDX, COLS);         \
    else if (D <= 32) LLMLAB_DELTA(32, MODE, GRIDX, COLS);    \
    else if (D <= 64) LLMLAB_DELTA(64, MODE, GRIDX, COLS);    \
    else if (D <= 128) LLMLAB_DELTA(128, MODE, GRIDX, COLS);  \
    else LLMLAB_DELTA(256, MODE, GRIDX, COLS);                \
  } while (0)
  LLMLAB_REQUIRE((E + 63) / 64 <= 65535 && (E + D + 63) / 64 <= 65535, "delta_scan: too many columns");
  if (chunk <= 0) {
    LLMLAB_DELTA_ANY(DELTA_WHOLE, n_reqs, E);
  } else {
    const int chunks = rows / chunk + n_reqs;
    LLMLAB_REQUIRE(chunk_state && chunk_trans && max_chunks >= chunks,
                   "delta_scan: %d rows of %d requests in chunks of %d need room for %d chunks, got %d", rows, n_reqs,
                   chunk, chunks, max_chunks);
    LLMLAB_REQUIRE(D <= 128, "delta_scan: chunks take states of up to 128 key channels, got %d", D);
    LLMLAB_DELTA_ANY(DELTA_LOCAL, chunks, E + D);
    const dim3 cgrid(n_reqs, n_heads, (E + CARRY_COLS - 1) / CARRY_COLS), cblock(64 * CARRY_GROUPS);
    if (D <= 16) hipLaunchKernelGGL(delta_carry_kernel<16>, cgrid, cblock, 0, stream, a);
    else if (D <= 32) hipLaunchKernelGGL(delta_carry_kernel<32>, cgrid, cblock, 0, stream, a);
    else if (D <= 64) hipLaunchKernelGGL(delta_carry_kernel<64>, cgrid, cblock, 0, stream, a);
    else hipLaunchKernelGGL(delta_carry_kernel<128>, cgrid, cblock, 0, stream, a);
    LLMLAB_DELTA_ANY(DELTA_FINISH, chunks, E);
  }
#undef LLMLAB_DELTA_ANY
#undef LLMLAB_DELTA
  LLMLAB_LAUNCH_CHECK("delta_scan");
  return 0;
}
