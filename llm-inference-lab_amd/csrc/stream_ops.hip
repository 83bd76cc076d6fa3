// Operations on the float32 residual stream around the sublayers of a layer, for gfx950:
//   embed_pairs     x[r] = norm(table[id] * scale + pairs[hash(previous id, id)])
//   causal_conv     out_t = h_t + sum_j w[:, j] h_(t - taps + 1 + j) over the positions of a request
//   norm_conv       the RMS norm of the stream's rows and that convolution over them in one launch
//   gated_add       x += y * sigmoid(gate + bias)
//   softcap         x = cap * tanh(x / cap)
//   rmsnorm_add     x += y / sqrt(mean(y^2) + eps) * w   (a norm on a sublayer's result, before the sum;
//                   the norm that reads the stream next may run in the same launch)
//   scaled_sum      out = a * y1 + b * y2
// What a request's earlier steps left (its last token, the last inputs of a convolution) lives in
// per-request slots; a step's rows of one request are adjacent.
#include "common.h"

extern "C" const char* llmlab_last_error() { return g_llmlab_error; }

// ------------------------------------------------------------------ embedding with hashed pairs
// One block a row.  The pair row of a sequence's first token is row `buckets`; else
// (previous * mul_prev + id * mul_cur) mod buckets, previous being the row before within the
// step or, for a request's first row of the step, previous_slot[slot].  The block of a
// request's first row also stores the request's LAST token of the step there, after it has read
// the old one (one thread does both, in that order; no other block touches the slot).
template <typename T>
__global__ __launch_bounds__(256) void embed_pairs_kernel(
    const T* __restrict__ table, const T* __restrict__ pairs, const int* __restrict__ ids,
    const int* __restrict__ positions, const int* __restrict__ row_req, const int* __restrict__ q_start,
    const int* __restrict__ req_rows, int* __restrict__ previous_slot, float scale, int vocab, int buckets,
    long long mul_prev, long long mul_cur, const void* __restrict__ norm_w, int norm_bf16, float eps,
    float* __restrict__ out, int hidden) {
  __shared__ float red[17];
  __shared__ int s_pair;
  const int r = blockIdx.x;
  int id = ids[r];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  if (threadIdx.x == 0) {
    int pair = -1;
    if (buckets > 0) {
      const int b = row_req[r], first = q_start[b];
      long long before = -1;
      if (r > first) {
        before = ids[r - 1];
      } else {
        const int slot = req_rows[b];
        before = previous_slot[slot];
        previous_slot[slot] = ids[q_start[b + 1] - 1];
      }
      if (before < 0) before = 0;
      pair = positions[r] == 0 ? buckets : (int)((before * mul_prev + (long long)id * mul_cur) % buckets);
    }
    s_pair = pair;
  }
  __syncthreads();
  const int pair = s_pair;
  const T* t = table + (size_t)id * hidden;
  const T* p = pair >= 0 ? pairs + (size_t)pair * hidden : nullptr;
  float* o = out + (size_t)r * hidden;
  float ss = 0.f;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    float v = to_float(t[c]) * scale;
    if (p) v += to_float(p[c]);
    o[c] = v;
    ss += v * v;
  }
  if (!norm_w) return;
  const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)hidden + eps);
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) o[c] = o[c] * inv * load_vec(norm_w, norm_bf16, c);
}

extern "C" int llmlab_embed_pairs(const void* table, const void* pairs, int dtype, const int* ids, const int* positions,
                                  const int* row_req, const int* q_start, const int* req_rows, int* previous_slot,
                                  float scale, int vocab, int buckets, long long mul_prev, long long mul_cur,
                                  const void* norm_w, int norm_dtype, float eps, float* out, int rows, int hidden,
                                  hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && hidden > 0 && vocab > 0 && buckets >= 0, "embed_pairs: bad sizes rows=%d hidden=%d", rows,
                 hidden);
  LLMLAB_REQUIRE(buckets == 0 || (pairs && positions && row_req && q_start && req_rows && previous_slot),
                 "embed_pairs: the pairs need their table, the step's description and the slots");
  if (rows == 0) return 0;
  if (dtype == DT_BF16)
    hipLaunchKernelGGL(embed_pairs_kernel<bf16_t>, dim3(rows), dim3(256), 0, stream, (const bf16_t*)table,
                       (const bf16_t*)pairs, ids, positions, row_req, q_start, req_rows, previous_slot, scale, vocab,
                       buckets, mul_prev, mul_cur, norm_w, norm_dtype == DT_BF16, eps, out, hidden);
  else
    hipLaunchKernelGGL(embed_pairs_kernel<float>, dim3(rows), dim3(256), 0, stream, (const float*)table,
                       (const float*)pairs, ids, positions, row_req, q_start, req_rows, previous_slot, scale, vocab,
                       buckets, mul_prev, mul_cur, norm_w, norm_dtype == DT_BF16, eps, out, hidden);
  LLMLAB_LAUNCH_CHECK("embed_pairs");
  return 0;
}

// ------------------------------------------------------------------ short causal convolution
// One block a row; a thread a channel.  Row r of request b (rows first .. first + n - 1 of the
// step) reads the rows r - back of the step while they belong to b, and state[slot][taps - 1 -
// (back - (r - first))] for the positions before the step (zeros before the sequence's start:
// a slot is zeroed when a request is admitted).  state: [slots, taps - 1, width].
template <typename T>
__global__ __launch_bounds__(256) void causal_conv_kernel(const T* __restrict__ h, const float* __restrict__ w, int taps,
                                                          const T* __restrict__ state, const int* __restrict__ row_req,
                                                          const int* __restrict__ q_start,
                                                          const int* __restrict__ req_rows, T* __restrict__ out,
                                                          int width) {
  const int r = blockIdx.x;
  const int b = row_req[r], first = q_start[b];
  const int inside = r - first;                       // rows of this request before r in the step
  const T* st = state ? state + (size_t)req_rows[b] * (taps - 1) * width : nullptr;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float own = to_float(h[(size_t)r * width + c]);
    float acc = own;
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;
      float v = 0.f;
      if (back == 0) v = own;
      else if (back <= inside) v = to_float(h[(size_t)(r - back) * width + c]);
      else if (st) v = to_float(st[(size_t)(taps - 1 - (back - inside)) * width + c]);
      acc = fmaf(w[(size_t)c * taps + j], v, acc);
    }
    out[(size_t)r * width + c] = from_float<T>(acc);
  }
}

// The slots after the step: the last taps - 1 inputs of the request, from what the slot held and
// the step's rows.  The block of a request's first row does it for the whole request; a thread
// reads place n + s before it writes place s, in rising order, so nothing is read after it changed.
template <typename T>
__global__ __launch_bounds__(256) void causal_conv_state_kernel(const T* __restrict__ h, int taps, T* __restrict__ state,
                                                                const int* __restrict__ row_req,
                                                                const int* __restrict__ q_start,
                                                                const int* __restrict__ req_rows, int width) {
  const int r = blockIdx.x;
  const int b = row_req[r], first = q_start[b];
  if (r != first) return;
  const int n = q_start[b + 1] - first, keep = taps - 1;
  T* st = state + (size_t)req_rows[b] * keep * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x)
    for (int s = 0; s < keep; ++s) {
      const int at = n + s;                    // place in [what the slot held | the step's rows]
      st[(size_t)s * width + c] = at < keep ? st[(size_t)at * width + c] : h[(size_t)(first + at - keep) * width + c];
    }
}

extern "C" int llmlab_causal_conv(const void* h, int dtype, const float* w, int taps, void* state, const int* row_req,
                                  const int* q_start, const int* req_rows, void* out, int rows, int width,
                                  hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && width > 0 && taps >= 1, "causal_conv: bad sizes rows=%d width=%d taps=%d", rows, width, taps);
  LLMLAB_REQUIRE(row_req && q_start && (taps == 1 || state == nullptr || req_rows),
                 "causal_conv: the step's description is missing");
  if (rows == 0) return 0;
  if (dtype == DT_BF16) {
    hipLaunchKernelGGL(causal_conv_kernel<bf16_t>, dim3(rows), dim3(256), 0, stream, (const bf16_t*)h, w, taps,
                       (const bf16_t*)state, row_req, q_start, req_rows, (bf16_t*)out, width);
    if (state && taps > 1)
      hipLaunchKernelGGL(causal_conv_state_kernel<bf16_t>, dim3(rows), dim3(256), 0, stream, (const bf16_t*)h, taps,
                         (bf16_t*)state, row_req, q_start, req_rows, width);
  } else {
    hipLaunchKernelGGL(causal_conv_kernel<float>, dim3(rows), dim3(256), 0, stream, (const float*)h, w, taps,
                       (const float*)state, row_req, q_start, req_rows, (float*)out, width);
    if (state && taps > 1)
      hipLaunchKernelGGL(causal_conv_state_kernel<float>, dim3(rows), dim3(256), 0, stream, (const float*)h, taps,
                         (float*)state, row_req, q_start, req_rows, width);
  }
  LLMLAB_LAUNCH_CHECK("causal_conv");
  return 0;
}

// ------------------------------------------------------------------ norm and convolution in one
// h = x / sqrt(mean(x^2) + eps) * g (rounded to T), conv = h + sum_j w[:, j] h_(t - taps + 1 + j):
// the RMS norm of the float32 stream's rows and the convolution over them in one launch.  One
// block a row.  A row's block norms the row itself and, again, the up to TAPS - 1 rows of its
// request before it in the step (the same sums in the same order as those rows' own blocks, so
// the same numbers); what lies before the step comes from the slots.  A thread takes NC_PER
// channels at a time, and every load of a round is unconditional (a row or a slot place that is
// not wanted is read at a place that is, and dropped), so that they travel together: a row
// that fits one round (width <= threads x NC_PER) costs one trip to memory, with the slot's
// inputs, the taps and the norm's weight asked for before the sums are reduced.  own_state:
// every request brings one row (row r is request r), and the row's block moves its slot on
// after it has read it (a thread owns its channels); otherwise causal_conv_state_kernel does
// that from h in a launch of its own.  NC_PER 1 serves few rows no wider than a block: the
// straight-line code of a block that runs once is fetched as it runs, and a quarter of the code
// is a quarter of that wait (8 rows of 896: 9.5 us with four channels a thread, 6.8 with one;
// the simplest kernels take 2.8).
template <typename T, int TAPS, int NC_PER>
struct NormConvLoads {
  float x[NC_PER][TAPS], s[NC_PER][TAPS], w[NC_PER][TAPS], g[NC_PER];
};

template <typename T, int TAPS, int NC_PER>
__device__ __forceinline__ void nc_load_x(NormConvLoads<T, TAPS, NC_PER>& v, const float* __restrict__ x, int r, int inside,
                                          int width, int c0, int stride) {
#pragma unroll
  for (int i = 0; i < NC_PER; ++i) {
    const int c = min(c0 + i * stride, width - 1);
#pragma unroll
    for (int k = 0; k < TAPS; ++k) v.x[i][k] = x[(size_t)(r - min(k, inside)) * width + c];
  }
}

template <typename T, int TAPS, int NC_PER>
__device__ __forceinline__ void nc_load_rest(NormConvLoads<T, TAPS, NC_PER>& v, const T* __restrict__ st, const float* __restrict__ w,
                                             const void* __restrict__ g, int g_bf16, int inside, int width, int c0,
                                             int stride) {
  constexpr int KEEP = TAPS - 1;
#pragma unroll
  for (int i = 0; i < NC_PER; ++i) {
    const int c = min(c0 + i * stride, width - 1);
    v.g[i] = load_vec(g, g_bf16, c);
#pragma unroll
    for (int k = 1; k < TAPS; ++k)                    // place in the slot of the input k positions back
      v.s[i][k] = st ? to_float(st[(size_t)min(max(KEEP - (k - inside), 0), KEEP - 1) * width + c]) : 0.f;
#pragma unroll
    for (int j = 0; j < TAPS; ++j) v.w[i][j] = w[(size_t)c * TAPS + j];
  }
}

template <typename T, int TAPS, int NC_PER>
__global__ __launch_bounds__(1024) void norm_conv_kernel(const float* __restrict__ x, const void* __restrict__ g,
                                                         int g_bf16, float eps, const float* __restrict__ w,
                                                         T* __restrict__ state, const int* __restrict__ row_req,
                                                         const int* __restrict__ q_start,
                                                         const int* __restrict__ req_rows, T* __restrict__ h,
                                                         T* __restrict__ conv, int width, int own_state) {
  constexpr int KEEP = TAPS - 1;
  __shared__ float red[16][TAPS];
  __shared__ float s_inv[TAPS];
  const int r = blockIdx.x;
  const int b = own_state ? r : row_req[r];
  const int first = own_state ? r : q_start[b];
  const int inside = min(r - first, KEEP);            // rows of this request before r that the taps reach
  T* st = state && KEEP > 0 ? state + (size_t)req_rows[b] * KEEP * width : nullptr;
  const int threads = blockDim.x, round = threads * NC_PER;
  const bool one_round = width <= round;
  NormConvLoads<T, TAPS, NC_PER> v;
  float ss[TAPS];
#pragma unroll
  for (int k = 0; k < TAPS; ++k) ss[k] = 0.f;
  for (int c0 = threadIdx.x; c0 < width; c0 += round) {
    nc_load_x<T, TAPS, NC_PER>(v, x, r, inside, width, c0, threads);
    if (one_round) nc_load_rest<T, TAPS, NC_PER>(v, st, w, g, g_bf16, inside, width, c0, threads);
#pragma unroll
    for (int i = 0; i < NC_PER; ++i)
      if (c0 + i * threads < width) {
#pragma unroll
        for (int k = 0; k < TAPS; ++k) ss[k] = fmaf(v.x[i][k], v.x[i][k], ss[k]);
      }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = threads >> 6;
#pragma unroll
  for (int k = 0; k < TAPS; ++k) ss[k] = wave_sum(ss[k]);
  if (lane == 0) {
#pragma unroll
    for (int k = 0; k < TAPS; ++k) red[wave][k] = ss[k];
  }
  __syncthreads();
  if (threadIdx.x < TAPS) {
    float t = 0.f;
    for (int i = 0; i < waves; ++i) t += red[i][threadIdx.x];
    s_inv[threadIdx.x] = 1.0f / sqrtf(t / (float)width + eps);
  }
  __syncthreads();
  float inv[TAPS];
#pragma unroll
  for (int k = 0; k < TAPS; ++k) inv[k] = s_inv[k];
  for (int c0 = threadIdx.x; c0 < width; c0 += round) {
    if (!one_round) {
      nc_load_x<T, TAPS, NC_PER>(v, x, r, inside, width, c0, threads);
      nc_load_rest<T, TAPS, NC_PER>(v, st, w, g, g_bf16, inside, width, c0, threads);
    }
#pragma unroll
    for (int i = 0; i < NC_PER; ++i) {
      const int c = c0 + i * threads;
      if (c >= width) continue;
      T hk[TAPS];
      hk[0] = from_float<T>(v.x[i][0] * inv[0] * v.g[i]);
      float acc = to_float(hk[0]);
      acc = fmaf(v.w[i][TAPS - 1], to_float(hk[0]), acc);
#pragma unroll
      for (int k = 1; k < TAPS; ++k) {
        hk[k] = k <= inside ? from_float<T>(v.x[i][k] * inv[k] * v.g[i]) : from_float<T>(v.s[i][k]);
        acc = fmaf(v.w[i][TAPS - 1 - k], to_float(hk[k]), acc);
      }
      h[(size_t)r * width + c] = hk[0];
      conv[(size_t)r * width + c] = from_float<T>(acc);
      if (own_state && st) {
#pragma unroll
        for (int s = 0; s < KEEP; ++s) st[(size_t)s * width + c] = hk[KEEP - 1 - s];
      }
    }
  }
}

template <typename T>
static void launch_norm_conv(int taps, int rows, hipStream_t stream, const float* x, const void* g, int g_bf16, float eps,
                             const float* w, T* state, const int* row_req, const int* q_start, const int* req_rows, T* h,
                             T* conv, int width, int own_state) {
  // few rows (a step bound by latency): a thread a channel up to a width of 1024, beyond that
  // four channels a thread in blocks of 1024; many rows: blocks of 256, of which a compute unit
  // holds several, four channels a thread
  int threads = 256, per = 4;
  if (rows <= 64 && width <= 1024) {
    per = 1;
    threads = (width + 63) / 64 * 64;
  } else if (rows <= 64) {
    while (threads < 1024 && threads * 4 < width) threads *= 2;
  }
#define LLMLAB_NORM_CONV(N)                                                                                               \
  case N:                                                                                                                 \
    if (per == 1)                                                                                                         \
      hipLaunchKernelGGL((norm_conv_kernel<T, N, 1>), dim3(rows), dim3(threads), 0, stream, x, g, g_bf16, eps, w, state,   \
                         row_req, q_start, req_rows, h, conv, width, own_state);                                          \
    else                                                                                                                  \
      hipLaunchKernelGGL((norm_conv_kernel<T, N, 4>), dim3(rows), dim3(threads), 0, stream, x, g, g_bf16, eps, w, state,   \
                         row_req, q_start, req_rows, h, conv, width, own_state);                                          \
    break;
  switch (taps) {
    LLMLAB_NORM_CONV(1) LLMLAB_NORM_CONV(2) LLMLAB_NORM_CONV(3) LLMLAB_NORM_CONV(4)
    LLMLAB_NORM_CONV(5) LLMLAB_NORM_CONV(6) LLMLAB_NORM_CONV(7) LLMLAB_NORM_CONV(8)
  }
#undef LLMLAB_NORM_CONV
}

// one_row_each: every request of the step brings exactly one row (the host knows).
extern "C" int llmlab_norm_conv(const float* x, const void* g, int g_dtype, float eps, const float* w, int taps,
                                void* state, const int* row_req, const int* q_start, const int* req_rows, void* h,
                                void* conv, int dtype, int rows, int width, int one_row_each, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && width > 0 && taps >= 1 && taps <= 8, "norm_conv: 1 to 8 taps, got rows=%d width=%d taps=%d",
                 rows, width, taps);
  LLMLAB_REQUIRE(row_req && q_start && (taps == 1 || (state && req_rows)), "norm_conv: the step's description is missing");
  if (rows == 0) return 0;
  if (dtype == DT_BF16) {
    launch_norm_conv<bf16_t>(taps, rows, stream, x, g, g_dtype == DT_BF16, eps, w, (bf16_t*)state, row_req, q_start,
                             req_rows, (bf16_t*)h, (bf16_t*)conv, width, one_row_each);
    if (taps > 1 && !one_row_each)
      hipLaunchKernelGGL(causal_conv_state_kernel<bf16_t>, dim3(rows), dim3(256), 0, stream, (const bf16_t*)h, taps,
                         (bf16_t*)state, row_req, q_start, req_rows, width);
  } else {
    launch_norm_conv<float>(taps, rows, stream, x, g, g_dtype == DT_BF16, eps, w, (float*)state, row_req, q_start,
                            req_rows, (float*)h, (float*)conv, width, one_row_each);
    if (taps > 1 && !one_row_each)
      hipLaunchKernelGGL(causal_conv_state_kernel<float>, dim3(rows), dim3(256), 0, stream, (const float*)h, taps,
                         (float*)state, row_req, q_start, req_rows, width);
  }
  LLMLAB_LAUNCH_CHECK("norm_conv");
  return 0;
}

// ------------------------------------------------------------------ gated sum into the stream
// x[r, c] += y[r, c] * sigmoid(gate[r, c or 0] + bias[c]); gate null: x += y.  All float32.
// y may come in `pieces` (a product left cut along its inner size): y = sum_s y[s * piece_stride + .],
// summed in the pieces' order.
__global__ void gated_add_kernel(float* __restrict__ x, const float* __restrict__ y, int pieces, size_t piece_stride,
                                 const float* __restrict__ gate, int gate_cols, const float* __restrict__ bias, int width,
                                 size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const size_t r = i / width;
    const int c = (int)(i - r * width);
    float v = y[i];
    for (int s = 1; s < pieces; ++s) v += y[s * piece_stride + i];
    if (gate) {
      float g = gate_cols == 1 ? gate[r] : gate[i];
      if (bias) g += bias[c];
      v = v / (1.f + __expf(-g));
    }
    x[i] += v;
  }
}

constexpr int GATED_ADD_MAX_PIECES = 8;
__global__ void gated_add4_kernel(floatx4* __restrict__ x, const floatx4* __restrict__ y, int pieces, size_t piece_stride4,
                                  const floatx4* __restrict__ gate, const floatx4* __restrict__ bias, int width4,
                                  size_t n4) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (size_t)gridDim.x * blockDim.x) {
    floatx4 g = gate[i];
    if (bias) g += bias[i % width4];
    floatx4 part[GATED_ADD_MAX_PIECES];            // (the pieces' loads together; past the last: the last again, dropped)
#pragma unroll
    for (int s = 0; s < GATED_ADD_MAX_PIECES; ++s) part[s] = y[(size_t)min(s, pieces - 1) * piece_stride4 + i];
    floatx4 v = part[0];
#pragma unroll
    for (int s = 1; s < GATED_ADD_MAX_PIECES; ++s)
      if (s < pieces) v += part[s];
    floatx4 o = x[i];
#pragma unroll
    for (int q = 0; q < 4; ++q) o[q] += v[q] / (1.f + __expf(-g[q]));
    x[i] = o;
  }
}

extern "C" int llmlab_gated_add(float* x, const float* y, int pieces, size_t piece_stride, const float* gate, int gate_cols,
                                const float* bias, int rows, int width, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && width > 0 && (gate == nullptr || gate_cols == 1 || gate_cols == width),
                 "gated_add: a gate per number or one per row, got %d columns for a width of %d", gate_cols, width);
  LLMLAB_REQUIRE(pieces >= 1 && pieces <= GATED_ADD_MAX_PIECES, "gated_add: 1 to %d pieces, got %d", GATED_ADD_MAX_PIECES,
                 pieces);
  const size_t n = (size_t)rows * width;
  if (n == 0) return 0;
  const bool vec = gate && gate_cols == width && width % 4 == 0 && piece_stride % 4 == 0 &&
                   (((uintptr_t)x | (uintptr_t)y | (uintptr_t)gate | (uintptr_t)bias) & 15) == 0;
  const size_t work = vec ? n / 4 : n;
  const int blocks = (int)((work + 255) / 256 < 65535 ? (work + 255) / 256 : 65535);
  if (vec)
    hipLaunchKernelGGL(gated_add4_kernel, dim3(blocks), dim3(256), 0, stream, (floatx4*)x, (const floatx4*)y, pieces,
                       piece_stride / 4, (const floatx4*)gate, (const floatx4*)bias, width / 4, n / 4);
  else
    hipLaunchKernelGGL(gated_add_kernel, dim3(blocks), dim3(256), 0, stream, x, y, pieces, piece_stride, gate, gate_cols,
                       bias, width, n);
  LLMLAB_LAUNCH_CHECK("gated_add");
  return 0;
}

// ------------------------------------------------------------------ norm of a sublayer's result into the stream
// One block a row: x[r, c] += v[c] / sqrt(mean(v^2) + eps) * w[c] with v = y[r] (or the sum of its
// pieces, in the pieces' order).  All float32.  A thread keeps up to NORM_ADD_KEEP of the row's numbers
// in registers between the two passes; wider rows are read again.
constexpr int NORM_ADD_KEEP = 8;
// NEXT: the norm that reads the stream next runs in the same launch on the row's new numbers:
// next_out[r, c] = T(x[r, c] / sqrt(mean(x[r]^2) + next_eps) * next_w[c]).
template <typename T, bool NEXT>
__global__ __launch_bounds__(256) void rmsnorm_add_kernel(float* __restrict__ x, const float* __restrict__ y, int pieces,
                                                          size_t piece_stride, const float* __restrict__ w, float eps,
                                                          int width, const float* __restrict__ next_w, float next_eps,
                                                          T* __restrict__ next_out) {
  __shared__ float red[17];
  const size_t row = (size_t)blockIdx.x * width;
  float keep[NORM_ADD_KEEP], xs[NORM_ADD_KEEP], ws[NORM_ADD_KEEP];
  float ss = 0.f;
  auto value = [&](int c) {
    float v = y[row + c];
    for (int s = 1; s < pieces; ++s) v += y[s * piece_stride + row + c];
    return v;
  };
  // (the stream's numbers and the weights are asked for together with the result's, before the
  // first sum is reduced: one trip to memory a row)
#pragma unroll
  for (int n = 0; n < NORM_ADD_KEEP; ++n) {
    const int c = threadIdx.x + 256 * n;
    keep[n] = c < width ? value(c) : 0.f;
    xs[n] = c < width ? x[row + c] : 0.f;
    ws[n] = c < width ? w[c] : 0.f;
    ss = fmaf(keep[n], keep[n], ss);
  }
  for (int c = threadIdx.x + 256 * NORM_ADD_KEEP; c < width; c += 256) {
    const float v = value(c);
    ss = fmaf(v, v, ss);
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)width + eps);
  float ss2 = 0.f;
#pragma unroll
  for (int n = 0; n < NORM_ADD_KEEP; ++n) {
    const int c = threadIdx.x + 256 * n;
    if (c < width) {
      keep[n] = xs[n] + keep[n] * inv * ws[n];
      x[row + c] = keep[n];
      ss2 = fmaf(keep[n], keep[n], ss2);
    }
  }
  for (int c = threadIdx.x + 256 * NORM_ADD_KEEP; c < width; c += 256) {
    const float v = x[row + c] + value(c) * inv * w[c];
    x[row + c] = v;
    ss2 = fmaf(v, v, ss2);
  }
  if (!NEXT) return;
  const float inv2 = 1.0f / sqrtf(block_sum(ss2, red) / (float)width + next_eps);
#pragma unroll
  for (int n = 0; n < NORM_ADD_KEEP; ++n) {
    const int c = threadIdx.x + 256 * n;
    if (c < width) next_out[row + c] = from_float<T>(keep[n] * inv2 * next_w[c]);
  }
  for (int c = threadIdx.x + 256 * NORM_ADD_KEEP; c < width; c += 256)      // (what this thread itself has just written)
    next_out[row + c] = from_float<T>(x[row + c] * inv2 * next_w[c]);
}

extern "C" int llmlab_rmsnorm_add(float* x, const float* y, int pieces, size_t piece_stride, const float* w, float eps,
                                  int rows, int width, const float* next_w, float next_eps, void* next_out,
                                  int next_dtype, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && width > 0 && pieces >= 1 && x && y && w, "rmsnorm_add: bad arguments rows=%d width=%d pieces=%d",
                 rows, width, pieces);
  LLMLAB_REQUIRE((next_w == nullptr) == (next_out == nullptr), "rmsnorm_add: the next norm needs its weight and its output");
  if (rows == 0) return 0;
  if (!next_out)
    hipLaunchKernelGGL((rmsnorm_add_kernel<float, false>), dim3(rows), dim3(256), 0, stream, x, y, pieces, piece_stride, w,
                       eps, width, nullptr, 0.f, nullptr);
  else if (next_dtype == DT_BF16)
    hipLaunchKernelGGL((rmsnorm_add_kernel<bf16_t, true>), dim3(rows), dim3(256), 0, stream, x, y, pieces, piece_stride, w,
                       eps, width, next_w, next_eps, (bf16_t*)next_out);
  else
    hipLaunchKernelGGL((rmsnorm_add_kernel<float, true>), dim3(rows), dim3(256), 0, stream, x, y, pieces, piece_stride, w,
                       eps, width, next_w, next_eps, (float*)next_out);
  LLMLAB_LAUNCH_CHECK("rmsnorm_add");
  return 0;
}

// ------------------------------------------------------------------ two results side by side
__global__ void scaled_sum_kernel(float* __restrict__ out, const float* __restrict__ y1, float a,
                                  const float* __restrict__ y2, float b, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    out[i] = a * y1[i] + b * y2[i];
}

extern "C" int llmlab_scaled_sum(float* out, const float* y1, float a, const float* y2, float b, size_t n,
                                 hipStream_t stream) {
  LLMLAB_REQUIRE(out && y1 && y2, "scaled_sum: null operand");
  if (n == 0) return 0;
  const int blocks = (int)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
  hipLaunchKernelGGL(scaled_sum_kernel, dim3(blocks), dim3(256), 0, stream, out, y1, a, y2, b, n);
  LLMLAB_LAUNCH_CHECK("scaled_sum");
  return 0;
}

// ------------------------------------------------------------------ soft cap
__global__ void softcap_kernel(float* __restrict__ x, float cap, float inv_cap, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    x[i] = cap * tanhf(x[i] * inv_cap);
}

extern "C" int llmlab_softcap(float* x, float cap, size_t n, hipStream_t stream) {
  LLMLAB_REQUIRE(cap > 0.f, "softcap: the cap must be positive, got %g", (double)cap);
  if (n == 0) return 0;
  const int blocks = (int)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
  hipLaunchKernelGGL(softcap_kernel, dim3(blocks), dim3(256), 0, stream, x, cap, 1.0f / cap, n);
  LLMLAB_LAUNCH_CHECK("softcap");
  return 0;
}
