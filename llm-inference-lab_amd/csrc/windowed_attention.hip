// Attention over a paged cache with a sliding window, a prefix of first positions that
// stays visible, and a softmax whose denominator holds one more, learned term per head
// (a "sink": a logit that only enlarges the denominator).  Keys and values may differ in width.  gfx950.
//
// Pages: keys [page, kv head, P, D] row by row; values [page, kv head, P, E] with the P * E
// numbers of a (page, kv head) in the order [P / 4][E][4]: the four keys of a quad side by
// side for each value channel, so that the sum over keys reads 8 bytes a lane (the matrix
// cores want runs of keys, the plain kernel four weights a load).
// Sizes are run-time arguments, so one library serves every head size.
#include "common.h"

extern "C" const char* llmlab_last_error() { return g_llmlab_error; }

constexpr float NEG_INF = -__builtin_huge_valf();

// where the value of the key at offset o of its page lies, channel e of E
__host__ __device__ inline size_t value_index(int o, int e, int E) { return ((size_t)(o >> 2) * E + e) * 4 + (o & 3); }

// --------------------------------------------------- projection -> q, cache
// One block per row of the step.  proj[r, :] holds the float32 projections of the row:
// q at column 0 (q_size = heads * D wide), then (if the layer has keys and values of its
// own) k (kv heads * D) and v (kv heads * E).  NORM: q and k are each divided by the root
// mean square over their WHOLE width (all heads together) and multiplied by a weight of
// that width, in float32.  q goes to q_out (compute dtype), k and v to the row's place
// in the pages.
template <typename T>
__global__ __launch_bounds__(256) void project_norm_write_kernel(
    const float* __restrict__ proj, int ld, int q_size, int k_size, int v_size, int norm, float eps,
    const float* __restrict__ q_w, const float* __restrict__ k_w, T* __restrict__ q_out,
    T* __restrict__ k_cache, T* __restrict__ v_cache, int n_kv, int D, int E, int page_size,
    const int* __restrict__ positions, const int* __restrict__ row_req, const int* __restrict__ table,
    int max_pages) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const float* src = proj + (size_t)r * ld;
  float inv_q = 1.f, inv_k = 1.f;
  if (norm) {
    float s = 0.f;
    for (int c = threadIdx.x; c < q_size; c += blockDim.x) s += src[c] * src[c];
    inv_q = 1.0f / sqrtf(block_sum(s, red) / (float)q_size + eps);
    if (k_size > 0) {
      s = 0.f;
      for (int c = threadIdx.x; c < k_size; c += blockDim.x) s += src[q_size + c] * src[q_size + c];
      inv_k = 1.0f / sqrtf(block_sum(s, red) / (float)k_size + eps);
    }
  }
  for (int c = threadIdx.x; c < q_size; c += blockDim.x)
    q_out[(size_t)r * q_size + c] = from_float<T>(norm ? src[c] * inv_q * q_w[c] : src[c]);
  if (k_size <= 0) return;
  const int pos = positions[r];
  const int page = table[(size_t)row_req[r] * max_pages + pos / page_size];
  const int slot = pos % page_size;
  for (int c = threadIdx.x; c < k_size; c += blockDim.x) {
    const int g = c / D, d = c - g * D;
    const float v = norm ? src[q_size + c] * inv_k * k_w[c] : src[q_size + c];
    k_cache[(((size_t)page * n_kv + g) * page_size + slot) * D + d] = from_float<T>(v);
  }
  for (int c = threadIdx.x; c < v_size; c += blockDim.x) {
    const int g = c / E, e = c - g * E;
    v_cache[((size_t)page * n_kv + g) * page_size * E + value_index(slot, e, E)] = from_float<T>(src[q_size + k_size + c]);
  }
}

extern "C" int llmlab_project_norm_write(const float* proj, int ld, int rows, int n_heads, int n_kv, int D, int E,
                                         int own_kv, int norm, float eps, const float* q_w, const float* k_w,
                                         void* q_out, void* k_cache, void* v_cache, int dtype, int page_size,
                                         const int* positions, const int* row_req, const int* table,
                                         int max_pages, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && n_heads > 0 && n_kv > 0 && D > 0 && E > 0 && page_size > 0,
                 "project_norm_write: bad sizes rows=%d heads=%d kv=%d D=%d E=%d page=%d", rows, n_heads, n_kv, D, E,
                 page_size);
  const int q_size = n_heads * D, k_size = own_kv ? n_kv * D : 0, v_size = own_kv ? n_kv * E : 0;
  LLMLAB_REQUIRE(ld >= q_size + k_size + v_size, "project_norm_write: rows of %d numbers do not hold %d", ld,
                 q_size + k_size + v_size);
  LLMLAB_REQUIRE(!norm || (q_w && (!own_kv || k_w)), "project_norm_write: the norm needs its weights");
  LLMLAB_REQUIRE(!own_kv || (k_cache && v_cache && positions && row_req && table),
                 "project_norm_write: keys and values need pages to go to");
  if (rows == 0) return 0;
  if (dtype == DT_BF16)
    hipLaunchKernelGGL(project_norm_write_kernel<bf16_t>, dim3(rows), dim3(256), 0, stream, proj, ld, q_size, k_size,
                       v_size, norm, eps, q_w, k_w, (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, n_kv, D, E,
                       page_size, positions, row_req, table, max_pages);
  else
    hipLaunchKernelGGL(project_norm_write_kernel<float>, dim3(rows), dim3(256), 0, stream, proj, ld, q_size, k_size,
                       v_size, norm, eps, q_w, k_w, (float*)q_out, (float*)k_cache, (float*)v_cache, n_kv, D, E,
                       page_size, positions, row_req, table, max_pages);
  LLMLAB_LAUNCH_CHECK("project_norm_write");
  return 0;
}

// The same for layers that turn their queries and keys by position and may mix their values
// with an earlier layer's.  proj[r, :] = q | k | v | gates (float32 sums); `bias` (float32, the
// same order, or null) is added first.  Rotation: of every query and key head the first rot_dims
// channels turn, channel 2i together with channel 2i + 1, by the angle positions[r] * freq[i]
// (float32), (u, v) -> (u cos - v sin, v cos + u sin), sine and cosine times `magnitude`; the
// other channels pass.  Values: mix 1 also leaves them, unrounded, in v_first[r]; mix 2 takes
// v <- (1 - lambda) v + lambda v_first[r] before they are stored.  The n_gate numbers behind the
// values go to gate_out [rows, n_gate] as they are.
constexpr int ROTATE_MAX_PAIRS = 256;
template <typename T>
__global__ __launch_bounds__(256) void project_rotate_write_kernel(
    const float* __restrict__ proj, int ld, int n_heads, int n_kv, int D, int E, const float* __restrict__ bias,
    const float* __restrict__ freq, int rot_dims, float magnitude, int mix, float lambda, float* __restrict__ v_first,
    int n_gate, float* __restrict__ gate_out, T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
    int page_size, const int* __restrict__ positions, const int* __restrict__ row_req, const int* __restrict__ table,
    int max_pages) {
  __shared__ float s_cos[ROTATE_MAX_PAIRS], s_sin[ROTATE_MAX_PAIRS];
  const int r = blockIdx.x;
  const float* src = proj + (size_t)r * ld;
  const int pos = positions[r];
  const int half = rot_dims >> 1;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float angle = (float)pos * freq[i];
    float sn, cs;
    sincosf(angle, &sn, &cs);
    s_cos[i] = cs * magnitude;
    s_sin[i] = sn * magnitude;
  }
  __syncthreads();
  const int q_size = n_heads * D, k_size = n_kv * D, v_size = n_kv * E;
  const int page = table[(size_t)row_req[r] * max_pages + pos / page_size];
  const int slot = pos % page_size;
  // queries and keys, a pair of channels a thread (D even where anything turns)
  const int pairs_per_head = (D + 1) >> 1;
  for (int p = threadIdx.x; p < (n_heads + n_kv) * pairs_per_head; p += blockDim.x) {
    const int hd = p / pairs_per_head, i = p - hd * pairs_per_head;
    const int c0 = hd * D + 2 * i;
    const bool two = 2 * i + 1 < D;
    float u = src[c0] + (bias ? bias[c0] : 0.f);
    float v = two ? src[c0 + 1] + (bias ? bias[c0 + 1] : 0.f) : 0.f;
    if (i < half) {
      const float cs = s_cos[i], sn = s_sin[i];
      const float u2 = u * cs - v * sn;
      v = v * cs + u * sn;
      u = u2;
    }
    if (hd < n_heads) {
      q_out[(size_t)r * q_size + c0] = from_float<T>(u);
      if (two) q_out[(size_t)r * q_size + c0 + 1] = from_float<T>(v);
    } else {
      const int g = hd - n_heads;
      T* dst = k_cache + (((size_t)page * n_kv + g) * page_size + slot) * D + 2 * i;
      dst[0] = from_float<T>(u);
      if (two) dst[1] = from_float<T>(v);
    }
  }
  for (int c = threadIdx.x; c < v_size; c += blockDim.x) {
    const int g = c / E, e = c - g * E;
    const int at = q_size + k_size + c;
    float v = src[at] + (bias ? bias[at] : 0.f);
    if (mix == 1) v_first[(size_t)r * v_size + c] = v;
    if (mix == 2) v = (1.f - lambda) * v + lambda * v_first[(size_t)r * v_size + c];
    v_cache[((size_t)page * n_kv + g) * page_size * E + value_index(slot, e, E)] = from_float<T>(v);
  }
  for (int c = threadIdx.x; c < n_gate; c += blockDim.x) {
    const int at = q_size + k_size + v_size + c;
    gate_out[(size_t)r * n_gate + c] = src[at] + (bias ? bias[at] : 0.f);
  }
}

extern "C" int llmlab_project_rotate_write(const float* proj, int ld, int rows, int n_heads, int n_kv, int D, int E,
                                           const float* bias, const float* freq, int rot_dims, float magnitude,
                                           int mix, float lambda, float* v_first, int n_gate, float* gate_out,
                                           void* q_out, void* k_cache, void* v_cache, int dtype, int page_size,
                                           const int* positions, const int* row_req, const int* table, int max_pages,
                                           hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && n_heads > 0 && n_kv > 0 && D > 0 && E > 0 && page_size > 0 && page_size % 4 == 0,
                 "project_rotate_write: bad sizes rows=%d heads=%d kv=%d D=%d E=%d page=%d", rows, n_heads, n_kv, D, E,
                 page_size);
  LLMLAB_REQUIRE(ld >= (n_heads + n_kv) * D + n_kv * E + n_gate && n_gate >= 0,
                 "project_rotate_write: rows of %d numbers do not hold the projections", ld);
  LLMLAB_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= D && rot_dims <= 2 * ROTATE_MAX_PAIRS &&
                 (rot_dims == 0 || freq), "project_rotate_write: %d of %d channels cannot turn in pairs", rot_dims, D);
  LLMLAB_REQUIRE(mix >= 0 && mix <= 2 && (mix == 0 || v_first), "project_rotate_write: mixed values need the first layer's");
  LLMLAB_REQUIRE(n_gate == 0 || gate_out, "project_rotate_write: gates need a place");
  LLMLAB_REQUIRE(q_out && k_cache && v_cache && positions && row_req && table,
                 "project_rotate_write: queries, pages, positions and the block table are needed");
  if (rows == 0) return 0;
  if (dtype == DT_BF16)
    hipLaunchKernelGGL(project_rotate_write_kernel<bf16_t>, dim3(rows), dim3(256), 0, stream, proj, ld, n_heads, n_kv, D, E,
                       bias, freq, rot_dims, magnitude, mix, lambda, v_first, n_gate, gate_out, (bf16_t*)q_out,
                       (bf16_t*)k_cache, (bf16_t*)v_cache, page_size, positions, row_req, table, max_pages);
  else
    hipLaunchKernelGGL(project_rotate_write_kernel<float>, dim3(rows), dim3(256), 0, stream, proj, ld, n_heads, n_kv, D, E,
                       bias, freq, rot_dims, magnitude, mix, lambda, v_first, n_gate, gate_out, (float*)q_out,
                       (float*)k_cache, (float*)v_cache, page_size, positions, row_req, table, max_pages);
  LLMLAB_LAUNCH_CHECK("project_rotate_write");
  return 0;
}

static int g_force_plain = 0;      // tests and measurements: no matrix-core kernel
extern "C" void llmlab_debug_windowed_attention_plain(int on) { g_force_plain = on; }
static int g_private_tiles = 0;    // tests and measurements: prompts by the kernel whose waves fetch their own tiles
extern "C" void llmlab_debug_windowed_attention_private_tiles(int on) { g_private_tiles = on; }

// ------------------------------------------------------------------ attention
// The query at position i of its request attends to the keys i - window < j <= i and to the
// kept prefix j < min(keep_first, i + 1); window <= 0: every j <= i.  Scores, the running maximum, the denominator
// and the weighted sum of values are float32.  With a sink the running maximum starts at
// sink[h] and the denominator at 1 = exp(sink - sink), and nothing is added to the weighted sum.
// mode 1 (MODE_SIGMOID): no softmax; the weight of a visible key is sigmoid(score + sink[h])
// (sink: then a bias per head added to every score, null for none), and the weights are not
// normalised.  The kernels then keep the running maximum at 0 and the denominator at 1, so the
// merge of shares and the final division stay as they are.
constexpr int MODE_SOFTMAX = 0, MODE_SIGMOID = 1;
__device__ __forceinline__ float sigmoid_weight(float s) { return 1.0f / (1.0f + __expf(-s)); }      // (-inf -> 0)
//
// Both kernels walk the keys in two runs, each from an aligned start, and mask key by key:
// the kept prefix [0, min(keep_first, B)) and [B, i], where B is the window's first key
// rounded down (to a quad of keys here, to 16 in the matrix-core kernel).
__device__ __forceinline__ bool sees(int i, int j, int window, int keep_first) {
  return j <= i && (window <= 0 || i - j < window || j < keep_first);
}

// ---- plain kernel: one wave per (row, head); float32 products.  Keys are taken 64 at a
// time: lane n scores one key (its own row of D numbers), the weights go through LDS, then
// lane e sums the values' channel e (and e + 64, ...) a quad of keys a load.
constexpr int MAX_E_PER_LANE = 16;     // value width up to 1024

template <typename T>
__device__ __forceinline__ float dot_row(const float* __restrict__ q, const T* __restrict__ k, int D);

template <>
__device__ __forceinline__ float dot_row<float>(const float* __restrict__ q, const float* __restrict__ k, int D) {
  float s = 0.f;
  if ((D & 3) == 0) {
    for (int d = 0; d < D; d += 4) {
      const floatx4 kv = *(const floatx4*)(k + d);
      s = fmaf(q[d], kv[0], s);
      s = fmaf(q[d + 1], kv[1], s);
      s = fmaf(q[d + 2], kv[2], s);
      s = fmaf(q[d + 3], kv[3], s);
    }
  } else {
    for (int d = 0; d < D; ++d) s = fmaf(q[d], k[d], s);
  }
  return s;
}

template <>
__device__ __forceinline__ float dot_row<bf16_t>(const float* __restrict__ q, const bf16_t* __restrict__ k, int D) {
  float s = 0.f;
  if ((D & 7) == 0) {
    for (int d = 0; d < D; d += 8) {
      const bf16x8 kv = *(const bf16x8*)(k + d);
#pragma unroll
      for (int j = 0; j < 8; ++j) s = fmaf(q[d + j], (float)kv[j], s);
    }
  } else {
    for (int d = 0; d < D; ++d) s = fmaf(q[d], (float)k[d], s);
  }
  return s;
}

__device__ __forceinline__ void load_quad(const float* p, float (&v)[4]) {
  const floatx4 t = *(const floatx4*)p;
  v[0] = t[0]; v[1] = t[1]; v[2] = t[2]; v[3] = t[3];
}
__device__ __forceinline__ void load_quad(const bf16_t* p, float (&v)[4]) {
  const bf16x4 t = *(const bf16x4*)p;
  v[0] = (float)t[0]; v[1] = (float)t[1]; v[2] = (float)t[2]; v[3] = (float)t[3];
}

template <typename T>
__global__ __launch_bounds__(64) void sink_window_attention_kernel(
    const T* __restrict__ q, int n_heads, int n_kv, int D, int E, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int* __restrict__ table, int max_pages, int page_size,
    const int* __restrict__ positions, const int* __restrict__ row_req, int window, int keep_first,
    const float* __restrict__ sink, float scale, T* __restrict__ out, const int* __restrict__ q_start, int long_from,
    int mode) {
  if (long_from > 0) {      // (rows of requests that bring many rows are the other kernel's)
    const int b = row_req[blockIdx.x];
    if (q_start[b + 1] - q_start[b] >= long_from) return;
  }
  extern __shared__ float lds[];       // q [D], weights [64], first value of each key's quad [64]
  float* qs = lds;
  float* ps = lds + D;
  size_t* vquad = (size_t*)(lds + D + 64 + ((D & 1) ? 1 : 0));
  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int g = h / (n_heads / n_kv);
  const int i = positions[r];
  const int* pages = table + (size_t)row_req[r] * max_pages;
  for (int d = lane; d < D; d += 64) qs[d] = to_float(q[((size_t)r * n_heads + h) * D + d]) * scale;
  __syncthreads();
  const int lo = window > 0 ? (i - window + 1 > 0 ? i - window + 1 : 0) : 0;
  const int b_start = lo & ~3;
  const int a_end = keep_first < b_start ? keep_first : b_start;
  const bool sig = mode == MODE_SIGMOID;
  const float bias = (sig && sink) ? sink[h] : 0.f;
  float m = sig ? 0.f : (sink ? sink[h] : NEG_INF);
  float l = (sig || sink) ? 1.f : 0.f;
  float acc[MAX_E_PER_LANE];
#pragma unroll
  for (int c = 0; c < MAX_E_PER_LANE; ++c) acc[c] = 0.f;
  for (int run = 0; run < 2; ++run) {
    const int first = run == 0 ? 0 : b_start;
    const int end = run == 0 ? a_end : i + 1;          // keys [first, end)
    for (int base = first; base < end; base += 64) {
      const int j = base + lane;
      const bool valid = j < end && sees(i, j, window, keep_first);
      float s = NEG_INF;
      if (j < end) {
        const int page = pages[j / page_size];
        const size_t head = ((size_t)page * n_kv + g) * page_size;
        if (valid) s = dot_row<T>(qs, k_cache + (head + (j % page_size)) * D, D);
        vquad[lane] = head * E + value_index(j % page_size, 0, E);       // (lanes 4 n are read below)
      }
      float p, corr;
      if (sig) {
        p = valid ? sigmoid_weight(s + bias) : 0.f;
        corr = 1.f;
      } else {
        const float m_new = fmaxf(m, wave_max(s));
        p = valid ? __expf(s - m_new) : 0.f;
        corr = (m == NEG_INF) ? 0.f : __expf(m - m_new);
        l = l * corr + wave_sum(p);
        m = m_new;
      }
      ps[lane] = p;
      __syncthreads();
      const int quads = ((end - base < 64 ? end - base : 64) + 3) >> 2;
#pragma unroll
      for (int c = 0; c < MAX_E_PER_LANE; ++c) {
        const int e = lane + 64 * c;
        if (e < E) {
          float a = acc[c] * corr;
          for (int t = 0; t < quads; ++t) {
            float v[4];
            load_quad(v_cache + vquad[4 * t] + (size_t)e * 4, v);
            a = fmaf(ps[4 * t], v[0], a);
            a = fmaf(ps[4 * t + 1], v[1], a);
            a = fmaf(ps[4 * t + 2], v[2], a);
            a = fmaf(ps[4 * t + 3], v[3], a);
          }
          acc[c] = a;
        }
      }
      __syncthreads();
    }
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int c = 0; c < MAX_E_PER_LANE; ++c) {
    const int e = lane + 64 * c;
    if (e < E) out[((size_t)r * n_heads + h) * E + e] = from_float<T>(acc[c] * inv);
  }
}

// ---- matrix-core kernels (bfloat16; D a multiple of 32, E of 16).  A wave serves 16 queries
// that share their keys: 16 consecutive rows of the step for one head (prompts), or the
// heads of one key/value head for one row (decoding: the keys are read once for the group).
// Keys come 32 at a time as two blocks of 16 (each within a page).  The scores are taken
// transposed, S^T = K Q^T, so that a lane ends up with the weights of ONE query for eight
// keys: exactly the operand the second product O^T = V^T P^T wants, with no trip through
// LDS.  Lane l = 16 g4 + c holds query c and, of a block of 16 keys, the keys 4 g4 .. 4 g4 + 3.
template <int EB>
struct Running {
  float m, l;
  floatx4 o[EB];
};

// The keys a wave's queries of one request can see, as a list of tiles of 32: first the kept
// prefix [0, a_end), then [b_start, p_hi] (p_lo, p_hi: the lowest and highest position among
// the queries; b_start: the lowest window's first key rounded down to 16).
struct KeyTiles {
  int a_end, b_start, end_b, tiles_a, tiles, p_lo, p_hi;
  __device__ KeyTiles(int p_lo_, int p_hi_, int window, int keep_first) : p_lo(p_lo_), p_hi(p_hi_) {
    const int lo = window > 0 ? (p_lo - window + 1 > 0 ? p_lo - window + 1 : 0) : 0;
    b_start = lo & ~15;
    a_end = keep_first < b_start ? keep_first : b_start;
    end_b = p_hi + 1;
    tiles_a = (a_end + 31) >> 5;
    tiles = tiles_a + ((end_b - b_start + 31) >> 5);
  }
};

// What a wave holds of one tile of 32 keys before the products: the keys' fragments of both
// blocks of 16, where the blocks' values start, and the tile's place.
template <int DC>
struct KeyFrags {
  bf16x8 k[2][DC];
  size_t vbase[2];
  bool have[2];
  int j0, end;
};

template <int DC, int E>
__device__ __forceinline__ void load_keys(KeyFrags<DC>& f, const KeyTiles& kt, int t, const int* __restrict__ pages,
                                          int page_size, int n_kv, int g, const bf16_t* __restrict__ k_cache) {
  constexpr int D = 32 * DC;
  const int lane = threadIdx.x & 63, c = lane & 15, g4 = lane >> 4;
  f.j0 = t < kt.tiles_a ? 32 * t : kt.b_start + 32 * (t - kt.tiles_a);
  f.end = t < kt.tiles_a ? kt.a_end : kt.end_b;
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int ju = f.j0 + 16 * u;
    f.have[u] = ju < f.end;
    f.vbase[u] = 0;
    if (f.have[u]) {
      const int page = pages[ju / page_size];
      const size_t head = ((size_t)page * n_kv + g) * page_size;
      const int off = ju % page_size;
      const bf16_t* kp = k_cache + (head + off + c) * D + 8 * g4;
#pragma unroll
      for (int dc = 0; dc < DC; ++dc) f.k[u][dc] = *(const bf16x8*)(kp + 32 * dc);
      f.vbase[u] = head * E + (size_t)((off >> 2) + g4) * E * 4;
    } else {
#pragma unroll
      for (int dc = 0; dc < DC; ++dc)
#pragma unroll
        for (int i = 0; i < 8; ++i) f.k[u][dc][i] = (bf16_t)0.f;
    }
  }
}

// Tiles [t_begin, t_end) of the list into the running softmax of the lane's query (position
// pos; seen: whether this lane's query takes part at all).  The loads run ahead of the
// products: a tile's values are asked for before its scores are taken, the next tile's keys
// before this tile's softmax.
template <int DC, int EB>
__device__ __forceinline__ void attend_tiles(const KeyTiles& kt, int t_begin, int t_end, const bf16x8 (&qf)[DC], bool seen,
                                             int pos, const int* __restrict__ pages, int page_size, int n_kv, int g,
                                             const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
                                             int window, int keep_first, float scale, Running<EB>& run,
                                             int mode, float bias) {
  constexpr int E = 16 * EB;
  const int lane = threadIdx.x & 63, c = lane & 15, g4 = lane >> 4;
  if (t_begin >= t_end) return;
  KeyFrags<DC> cur, nxt;
  load_keys<DC, E>(cur, kt, t_begin, pages, page_size, n_kv, g, k_cache);
  for (int t = t_begin; t < t_end; ++t) {
    bf16x8 vf[EB];
#pragma unroll
    for (int eb = 0; eb < EB; ++eb)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        bf16x4 quad = bf16x4{(bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f};
        if (cur.have[u]) quad = *(const bf16x4*)(v_cache + cur.vbase[u] + (size_t)(16 * eb + c) * 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) vf[eb][4 * u + i] = quad[i];
      }
    if (t + 1 < t_end) load_keys<DC, E>(nxt, kt, t + 1, pages, page_size, n_kv, g, k_cache);
    floatx4 s[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      s[u] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int dc = 0; dc < DC; ++dc)
        s[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.k[u][dc], qf[dc], s[u], 0, 0, 0);
    }
    float tmax = NEG_INF;
    // a whole tile that every query of the wave sees (behind the lowest position, inside the
    // window of the highest or the kept prefix) needs no mask key by key: most tiles of a long window
    const bool interior = cur.have[1] && cur.j0 + 31 < cur.end && cur.j0 + 31 <= kt.p_lo &&
                          (window <= 0 || kt.p_hi - cur.j0 < window || cur.j0 + 31 < keep_first);
    if (interior) {
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          s[u][i] = seen ? s[u][i] * scale : NEG_INF;
          tmax = fmaxf(tmax, s[u][i]);
        }
    } else {
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int j = cur.j0 + 16 * u + 4 * g4 + i;
          const bool ok = cur.have[u] && seen && j < cur.end && sees(pos, j, window, keep_first);
          s[u][i] = ok ? s[u][i] * scale : NEG_INF;
          tmax = fmaxf(tmax, s[u][i]);
        }
    }
    bf16x8 pf;
    if (mode == MODE_SIGMOID) {
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) pf[4 * u + i] = (bf16_t)sigmoid_weight(s[u][i] + bias);      // (masked: -inf -> 0)
#pragma unroll
      for (int eb = 0; eb < EB; ++eb)
        run.o[eb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[eb], pf, run.o[eb], 0, 0, 0);
    } else {
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, WAVE));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
    const float m_new = fmaxf(run.m, tmax);
    const float m_use = m_new == NEG_INF ? 0.f : m_new;
    const float corr = run.m == NEG_INF ? 0.f : __expf(run.m - m_use);
    float sum = 0.f;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = __expf(s[u][i] - m_use);       // (exp(-inf) = 0 for a masked key)
        sum += p;
        pf[4 * u + i] = (bf16_t)p;
      }
    sum += __shfl_xor(sum, 16, WAVE);
    sum += __shfl_xor(sum, 32, WAVE);
    run.l = run.l * corr + sum;
    run.m = m_new;
#pragma unroll
    for (int eb = 0; eb < EB; ++eb) {
#pragma unroll
      for (int i = 0; i < 4; ++i) run.o[eb][i] *= corr;
      run.o[eb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[eb], pf, run.o[eb], 0, 0, 0);
    }
    }
    cur = nxt;
  }
}

struct MfmaArgs {
  const bf16_t* q; int n_rows, n_heads, n_kv;
  const bf16_t* k_cache; const bf16_t* v_cache; const int* table; int max_pages, page_size;
  const int* positions; const int* row_req; int window, keep_first; const float* sink; float scale;
  bf16_t* out; const int* q_start; int long_from;
  int splits; float* part_o; float* part_ml;      // (decoding) [rows, heads, splits, E] and [rows, heads, splits, 2]
  int mode;                                       // MODE_SOFTMAX, or MODE_SIGMOID (sink: the bias of the scores)
};

// Prompts: a wave takes 16 consecutive rows and one head, a block four such tiles.  Rows of
// several requests in one tile are served request after request (the others' columns masked).
template <int DC, int EB>
__global__ __launch_bounds__(256) void sink_window_attention_mfma_kernel(MfmaArgs a) {
  constexpr int D = 32 * DC, E = 16 * EB;
  const int lane = threadIdx.x & 63, c = lane & 15, g4 = lane >> 4;
  const int r0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * 16;
  if (r0 >= a.n_rows) return;
  const int h = blockIdx.y, g = h / (a.n_heads / a.n_kv);
  const int r = r0 + c;
  const bool row_ok = r < a.n_rows;
  const int pos = row_ok ? a.positions[r] : 0;
  const int req = row_ok ? a.row_req[r] : -1;
  bf16x8 qf[DC];
#pragma unroll
  for (int dc = 0; dc < DC; ++dc) {
    if (row_ok) qf[dc] = *(const bf16x8*)(a.q + ((size_t)r * a.n_heads + h) * D + 32 * dc + 8 * g4);
    else
#pragma unroll
      for (int i = 0; i < 8; ++i) qf[dc][i] = (bf16_t)0.f;
  }
  Running<EB> run;
  const bool sig = a.mode == MODE_SIGMOID;
  const float bias = (sig && a.sink) ? a.sink[h] : 0.f;
  run.m = sig ? 0.f : (a.sink ? a.sink[h] : NEG_INF);
  run.l = (sig || a.sink) ? 1.f : 0.f;
#pragma unroll
  for (int eb = 0; eb < EB; ++eb) run.o[eb] = floatx4{0.f, 0.f, 0.f, 0.f};
  const int b_first = __builtin_amdgcn_readfirstlane(a.row_req[r0]);
  const int b_last = __builtin_amdgcn_readfirstlane(a.row_req[(r0 + 15 < a.n_rows ? r0 + 15 : a.n_rows - 1)]);
  for (int b = b_first; b <= b_last; ++b) {
    if (a.long_from > 0 && a.q_start[b + 1] - a.q_start[b] < a.long_from) continue;      // (the other kernels' rows)
    const bool mine = req == b;
    int p_lo = mine ? pos : 0x7fffffff, p_hi = mine ? pos : -1;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      p_lo = min(p_lo, __shfl_xor(p_lo, off, WAVE));
      p_hi = max(p_hi, __shfl_xor(p_hi, off, WAVE));
    }
    if (p_hi < 0) continue;
    const KeyTiles kt(p_lo, p_hi, a.window, a.keep_first);
    attend_tiles<DC, EB>(kt, 0, kt.tiles, qf, mine, pos, a.table + (size_t)b * a.max_pages, a.page_size, a.n_kv, g,
                         a.k_cache, a.v_cache, a.window, a.keep_first, a.scale, run, a.mode, bias);
  }
  if (!row_ok) return;
  if (a.long_from > 0 && a.q_start[req + 1] - a.q_start[req] < a.long_from) return;
  const float inv = 1.0f / run.l;
#pragma unroll
  for (int eb = 0; eb < EB; ++eb) {
    bf16x4 w;
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (bf16_t)(run.o[eb][i] * inv);
    *(bf16x4*)(a.out + ((size_t)r * a.n_heads + h) * E + 16 * eb + 4 * g4) = w;
  }
}

// Prompts whose heads read the same keys and values (one key/value head, or groups of a multiple
// of four heads): a block takes 16 consecutive rows and FOUR heads, a wave a head.  The block
// stages every tile of 32 keys and their values in LDS once (each thread asks for its 16-byte
// pieces two tiles ahead and stores them a tile ahead), and the waves take their fragments from
// there instead of each from L2.  Key rows lie 16 bytes apart from a
// multiple of 256 bytes and the values' quad rows 128, so that the lanes of a read spread over the
// banks.  Everything else (the list of tiles, masks, the running softmax, the transposed
// products) is the kernel's above; all waves of a block walk the same tiles, so the barriers
// are reached by all.
template <int DC, int EB>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void sink_window_attention_shared_kernel(MfmaArgs a) {
  constexpr int D = 32 * DC, E = 16 * EB;
  constexpr int KROW = D + 8, VROW = 4 * E + 64;
  constexpr int KCHUNKS = 4 * D, VCHUNKS = 4 * E;            // 16-byte pieces of a tile's keys / values
  constexpr int KCH = (KCHUNKS + 255) / 256, VCH = (VCHUNKS + 255) / 256;
  __shared__ __attribute__((aligned(16))) bf16_t ks[2 * 16 * KROW];
  __shared__ __attribute__((aligned(16))) bf16_t vs[2 * 4 * VROW];
  const int tid = threadIdx.x, lane = tid & 63, c = lane & 15, g4 = lane >> 4, wave = tid >> 6;
  const int r0 = blockIdx.x * 16;
  if (r0 >= a.n_rows) return;
  const int h_raw = blockIdx.y * 4 + wave;
  const bool head_ok = h_raw < a.n_heads;
  const int h = head_ok ? h_raw : a.n_heads - 1;
  const int g = (blockIdx.y * 4) / (a.n_heads / a.n_kv);
  const int r = r0 + c;
  const bool row_ok = r < a.n_rows;
  const int pos = row_ok ? a.positions[r] : 0;
  const int req = row_ok ? a.row_req[r] : -1;
  bf16x8 zero8;
#pragma unroll
  for (int i = 0; i < 8; ++i) zero8[i] = (bf16_t)0.f;
  bf16x8 qf[DC];
#pragma unroll
  for (int dc = 0; dc < DC; ++dc)
    qf[dc] = row_ok ? *(const bf16x8*)(a.q + ((size_t)r * a.n_heads + h) * D + 32 * dc + 8 * g4) : zero8;
  Running<EB> run;
  const bool sig = a.mode == MODE_SIGMOID;
  const float bias = (sig && a.sink) ? a.sink[h] : 0.f;
  run.m = sig ? 0.f : (a.sink ? a.sink[h] : NEG_INF);
  run.l = (sig || a.sink) ? 1.f : 0.f;
#pragma unroll
  for (int eb = 0; eb < EB; ++eb) run.o[eb] = floatx4{0.f, 0.f, 0.f, 0.f};
  const int b_first = __builtin_amdgcn_readfirstlane(a.row_req[r0]);
  const int b_last = __builtin_amdgcn_readfirstlane(a.row_req[(r0 + 15 < a.n_rows ? r0 + 15 : a.n_rows - 1)]);
  for (int b = b_first; b <= b_last; ++b) {
    if (a.long_from > 0 && a.q_start[b + 1] - a.q_start[b] < a.long_from) continue;      // (the other kernels' rows)
    const bool mine = req == b;
    int p_lo = mine ? pos : 0x7fffffff, p_hi = mine ? pos : -1;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      p_lo = min(p_lo, __shfl_xor(p_lo, off, WAVE));
      p_hi = max(p_hi, __shfl_xor(p_hi, off, WAVE));
    }
    if (p_hi < 0) continue;
    const KeyTiles kt(p_lo, p_hi, a.window, a.keep_first);
    const int* pages = a.table + (size_t)b * a.max_pages;
    // Two sets of staging registers: a tile's pieces are asked for TWO tiles ahead and stored one
    // tile ahead, so that their way from memory lies behind the products of a whole tile and
    // more (the longest block's tiles, one after the other, are what a prompt's attention takes).
    bf16x8 k_a[KCH], v_a[VCH], k_b[KCH], v_b[VCH];
    // the 16-byte pieces of tile t that this thread brings
    auto fetch = [&](int t, bf16x8 (&kreg)[KCH], bf16x8 (&vreg)[VCH]) {
      const int j0 = t < kt.tiles_a ? 32 * t : kt.b_start + 32 * (t - kt.tiles_a);
      const int end = t < kt.tiles_a ? kt.a_end : kt.end_b;
      size_t kbase[2], vbase[2];
      bool have[2];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int ju = j0 + 16 * u;
        have[u] = ju < end;
        kbase[u] = vbase[u] = 0;
        if (have[u]) {
          const int page = pages[ju / a.page_size];
          const size_t head = ((size_t)page * a.n_kv + g) * a.page_size;
          const int off = ju % a.page_size;
          kbase[u] = (head + off) * D;
          vbase[u] = head * E + (size_t)(off >> 2) * E * 4;
        }
      }
#pragma unroll
      for (int i = 0; i < KCH; ++i) {
        const int idx = tid + 256 * i;
        const int u = idx / (2 * D), rem = idx % (2 * D);
        kreg[i] = (idx < KCHUNKS && have[u & 1]) ? *(const bf16x8*)(a.k_cache + kbase[u & 1] + (size_t)rem * 8) : zero8;
      }
#pragma unroll
      for (int i = 0; i < VCH; ++i) {
        const int idx = tid + 256 * i;
        const int u = idx / (2 * E), rem = idx % (2 * E);
        vreg[i] = (idx < VCHUNKS && have[u & 1]) ? *(const bf16x8*)(a.v_cache + vbase[u & 1] + (size_t)rem * 8) : zero8;
      }
    };
    auto stash = [&](const bf16x8 (&kreg)[KCH], const bf16x8 (&vreg)[VCH]) {
#pragma unroll
      for (int i = 0; i < KCH; ++i) {
        const int idx = tid + 256 * i;
        if (idx < KCHUNKS) {
          const int u = idx / (2 * D), rem = idx % (2 * D);
          const int key = rem / (D / 8), part = rem % (D / 8);
          *(bf16x8*)(ks + (u * 16 + key) * KROW + part * 8) = kreg[i];
        }
      }
#pragma unroll
      for (int i = 0; i < VCH; ++i) {
        const int idx = tid + 256 * i;
        if (idx < VCHUNKS) {
          const int u = idx / (2 * E), rem = idx % (2 * E);
          const int quad = rem / (E / 2), within = rem % (E / 2);
          *(bf16x8*)(vs + (u * 4 + quad) * VROW + within * 8) = vreg[i];
        }
      }
    };
    // tile t, which lies in LDS, into the running softmax
    auto attend = [&](int t) {
      const int j0 = t < kt.tiles_a ? 32 * t : kt.b_start + 32 * (t - kt.tiles_a);
      const int end = t < kt.tiles_a ? kt.a_end : kt.end_b;
      const bool have1 = j0 + 16 < end;
      floatx4 s[2];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        s[u] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dc = 0; dc < DC; ++dc) {
          const bf16x8 kf = *(const bf16x8*)(ks + (u * 16 + c) * KROW + 32 * dc + 8 * g4);
          s[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[dc], s[u], 0, 0, 0);
        }
      }
      float tmax = NEG_INF;
      const bool interior = have1 && j0 + 31 < end && j0 + 31 <= kt.p_lo &&
                            (a.window <= 0 || kt.p_hi - j0 < a.window || j0 + 31 < a.keep_first);
      if (interior) {
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            s[u][i] = mine ? s[u][i] * a.scale : NEG_INF;
            tmax = fmaxf(tmax, s[u][i]);
          }
      } else {
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int j = j0 + 16 * u + 4 * g4 + i;
            const bool ok = mine && j < end && sees(pos, j, a.window, a.keep_first);
            s[u][i] = ok ? s[u][i] * a.scale : NEG_INF;
            tmax = fmaxf(tmax, s[u][i]);
          }
      }
      float corr = 1.f;
      bf16x8 pf;
      if (a.mode == MODE_SIGMOID) {
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int i = 0; i < 4; ++i) pf[4 * u + i] = (bf16_t)sigmoid_weight(s[u][i] + bias);      // (masked: -inf -> 0)
      } else {
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, WAVE));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
      const float m_new = fmaxf(run.m, tmax);
      const float m_use = m_new == NEG_INF ? 0.f : m_new;
      corr = run.m == NEG_INF ? 0.f : __expf(run.m - m_use);
      float sum = 0.f;
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float p = __expf(s[u][i] - m_use);       // (exp(-inf) = 0 for a masked key)
          sum += p;
          pf[4 * u + i] = (bf16_t)p;
        }
      sum += __shfl_xor(sum, 16, WAVE);
      sum += __shfl_xor(sum, 32, WAVE);
      run.l = run.l * corr + sum;
      run.m = m_new;
      }
#pragma unroll
      for (int eb = 0; eb < EB; ++eb) {
        bf16x8 vf;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const bf16x4 quad = *(const bf16x4*)(vs + (u * 4 + g4) * VROW + (16 * eb + c) * 4);
#pragma unroll
          for (int i = 0; i < 4; ++i) vf[4 * u + i] = quad[i];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) run.o[eb][i] *= corr;
        run.o[eb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, run.o[eb], 0, 0, 0);
      }
    };
    const int T = kt.tiles;
    __syncthreads();                                  // (the request before this one has been read)
    fetch(0, k_a, v_a);
    stash(k_a, v_a);
    __syncthreads();
    if (T > 1) fetch(1, k_a, v_a);
    for (int t = 0; t < T; t += 2) {
      // tile t lies in LDS, tile t + 1 is on its way into set a
      if (t + 2 < T) fetch(t + 2, k_b, v_b);
      attend(t);
      __syncthreads();                                // (every wave has read the tile)
      if (t + 1 < T) stash(k_a, v_a);
      __syncthreads();
      if (t + 1 >= T) break;
      // tile t + 1 lies in LDS, tile t + 2 is on its way into set b
      if (t + 3 < T) fetch(t + 3, k_a, v_a);
      attend(t + 1);
      __syncthreads();
      if (t + 2 < T) stash(k_b, v_b);
      __syncthreads();
    }
  }
  if (!row_ok || !head_ok) return;
  if (a.long_from > 0 && a.q_start[req + 1] - a.q_start[req] < a.long_from) return;
  const float inv = 1.0f / run.l;
#pragma unroll
  for (int eb = 0; eb < EB; ++eb) {
    bf16x4 w;
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (bf16_t)(run.o[eb][i] * inv);
    *(bf16x4*)(a.out + ((size_t)r * a.n_heads + h) * E + 16 * eb + 4 * g4) = w;
  }
}

// Decoding (requests that bring fewer than long_from rows): a wave takes ONE row, the heads of
// one key/value head (16 at a time) and one of `splits` shares of the row's key tiles, so that
// few rows still fill the chip.  With one share the result is final; else the share's
// maximum, denominator and unnormalised sum go to part_ml / part_o for the merge kernel.
// The sink enters the first share only.
template <int DC, int EB>
__global__ __launch_bounds__(64) void sink_window_attention_grouped_kernel(MfmaArgs a) {
  constexpr int D = 32 * DC, E = 16 * EB;
  const int lane = threadIdx.x & 63, c = lane & 15, g4 = lane >> 4;
  const int r = blockIdx.x;
  const int b = a.row_req[r];
  if (a.long_from > 0 && a.q_start[b + 1] - a.q_start[b] >= a.long_from) return;      // (the prompts' kernel's rows)
  const int group = a.n_heads / a.n_kv, per_group = (group + 15) >> 4;
  const int g = blockIdx.y / per_group;
  const int hc = (blockIdx.y % per_group) * 16 + c;        // this lane's head within the group
  const bool head_ok = hc < group;
  const int h = g * group + hc;
  const int pos = a.positions[r];
  bf16x8 qf[DC];
#pragma unroll
  for (int dc = 0; dc < DC; ++dc) {
    if (head_ok) qf[dc] = *(const bf16x8*)(a.q + ((size_t)r * a.n_heads + h) * D + 32 * dc + 8 * g4);
    else
#pragma unroll
      for (int i = 0; i < 8; ++i) qf[dc][i] = (bf16_t)0.f;
  }
  const int z = blockIdx.z;
  Running<EB> run;
  const bool sig = a.mode == MODE_SIGMOID;
  const float bias = (sig && a.sink && head_ok) ? a.sink[h] : 0.f;
  run.m = sig ? 0.f : ((a.sink && head_ok && z == 0) ? a.sink[h] : NEG_INF);
  run.l = sig ? (z == 0 ? 1.f : 0.f) : ((a.sink && head_ok && z == 0) ? 1.f : 0.f);
#pragma unroll
  for (int eb = 0; eb < EB; ++eb) run.o[eb] = floatx4{0.f, 0.f, 0.f, 0.f};
  const KeyTiles kt(pos, pos, a.window, a.keep_first);
  const int per = (kt.tiles + a.splits - 1) / a.splits;
  const int t_begin = z * per, t_end = (z + 1) * per < kt.tiles ? (z + 1) * per : kt.tiles;
  attend_tiles<DC, EB>(kt, t_begin, t_end, qf, head_ok, pos, a.table + (size_t)b * a.max_pages, a.page_size, a.n_kv, g,
                       a.k_cache, a.v_cache, a.window, a.keep_first, a.scale, run, a.mode, bias);
  if (!head_ok) return;
  if (a.splits == 1) {
    const float inv = 1.0f / run.l;
#pragma unroll
    for (int eb = 0; eb < EB; ++eb) {
      bf16x4 w;
#pragma unroll
      for (int i = 0; i < 4; ++i) w[i] = (bf16_t)(run.o[eb][i] * inv);
      *(bf16x4*)(a.out + ((size_t)r * a.n_heads + h) * E + 16 * eb + 4 * g4) = w;
    }
    return;
  }
  const size_t share = ((size_t)r * a.n_heads + h) * a.splits + z;
  if (g4 == 0) {
    a.part_ml[share * 2] = run.m;
    a.part_ml[share * 2 + 1] = run.l;
  }
#pragma unroll
  for (int eb = 0; eb < EB; ++eb) *(floatx4*)(a.part_o + share * E + 16 * eb + 4 * g4) = run.o[eb];
}

// out[r, h] = sum_z exp(m_z - M) o_z / sum_z exp(m_z - M) l_z over the shares of the row's keys.
// One wave per (row, head).  The shares' maxima and sums are read once, a lane a share; the
// shares' weights exp(m_z - M) lie in LDS, and the loop over the shares' partial outputs has no
// branch (an empty share weighs zero and its numbers are dropped), so its loads travel together.
constexpr int MERGE_MAX_SPLITS = 256;
__global__ __launch_bounds__(64) void sink_window_attention_merge_kernel(MfmaArgs a, int E) {
  __shared__ float s_w[MERGE_MAX_SPLITS];
  const int r = blockIdx.x, h = blockIdx.y;
  const int b = a.row_req[r];
  if (a.long_from > 0 && a.q_start[b + 1] - a.q_start[b] >= a.long_from) return;
  const size_t first = ((size_t)r * a.n_heads + h) * a.splits;
  constexpr int PER_LANE = MERGE_MAX_SPLITS / 64;
  float m[PER_LANE], l[PER_LANE];
  float big = NEG_INF;
#pragma unroll
  for (int i = 0; i < PER_LANE; ++i) {
    const int z = threadIdx.x + 64 * i;
    const int at = min(z, a.splits - 1);
    const float mz = a.part_ml[(first + at) * 2], lz = a.part_ml[(first + at) * 2 + 1];
    m[i] = z < a.splits ? mz : NEG_INF;
    l[i] = lz;
    big = fmaxf(big, m[i]);
  }
  big = wave_max(big);
  float den = 0.f;
#pragma unroll
  for (int i = 0; i < PER_LANE; ++i) {
    const float w = m[i] != NEG_INF ? __expf(m[i] - big) : 0.f;
    if (w != 0.f) den = fmaf(w, l[i], den);
    s_w[threadIdx.x + 64 * i] = w;
  }
  den = wave_sum(den);
  __syncthreads();
  const float inv = 1.0f / den;
  for (int e = threadIdx.x; e < E; e += 64) {
    float acc = 0.f;
    int z = 0;
    for (; z + 4 <= a.splits; z += 4) {
      float o[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = a.part_o[(first + z + j) * E + e];
#pragma unroll
      for (int j = 0; j < 4; ++j) acc = fmaf(s_w[z + j], s_w[z + j] != 0.f ? o[j] : 0.f, acc);
    }
    for (; z < a.splits; ++z) {
      const float o = a.part_o[(first + z) * E + e];
      acc = fmaf(s_w[z], s_w[z] != 0.f ? o : 0.f, acc);
    }
    a.out[((size_t)r * a.n_heads + h) * E + e] = (bf16_t)(acc * inv);
  }
}


// Whether the matrix-core kernel takes these sizes at all.
extern "C" int llmlab_sink_window_attention_has_mfma(int dtype, int D, int E, int page_size) {
  if (g_force_plain || dtype != DT_BF16 || D % 32 != 0 || E % 16 != 0 || page_size % 16 != 0) return 0;
  // (keys and values up to 128 wide in any combination; values of 192 and 256 beside keys of 64 to
  // 128; wider keys, up to 256, where both are of one width: the latent form, whose values are its keys)
  return (D <= 128 && E <= 128) || (D >= 64 && D <= 128 && (E == 192 || E == 256)) || (D == E && D <= 256);
}

template <int DC>
static void launch_mfma(int EBv, int which, dim3 grid, dim3 block, hipStream_t stream, const MfmaArgs& a) {
#define LLMLAB_MFMA(EBC)                                                                                      \
  case EBC:                                                                                                   \
    if (which == 0) hipLaunchKernelGGL((sink_window_attention_mfma_kernel<DC, EBC>), grid, block, 0, stream, a); \
    else if (which == 2) hipLaunchKernelGGL((sink_window_attention_shared_kernel<DC, EBC>), grid, block, 0, stream, a); \
    else hipLaunchKernelGGL((sink_window_attention_grouped_kernel<DC, EBC>), grid, block, 0, stream, a);      \
    break;
  switch (EBv) {
    LLMLAB_MFMA(1) LLMLAB_MFMA(2) LLMLAB_MFMA(3) LLMLAB_MFMA(4) LLMLAB_MFMA(5) LLMLAB_MFMA(6) LLMLAB_MFMA(7) LLMLAB_MFMA(8)
  }
  if constexpr (DC >= 2) {      // (values of 192 and 256 beside keys of 64 to 128)
    switch (EBv) { LLMLAB_MFMA(12) LLMLAB_MFMA(16) }
  }
#undef LLMLAB_MFMA
}

static void launch_mfma_any(int D, int E, int which, dim3 grid, dim3 block, hipStream_t stream, const MfmaArgs& a) {
#define LLMLAB_MFMA_SQUARE(DCV)                                                                                          \
  case DCV:                                                                                                             \
    if (which == 0) hipLaunchKernelGGL((sink_window_attention_mfma_kernel<DCV, 2 * DCV>), grid, block, 0, stream, a);     \
    else if (which == 2) hipLaunchKernelGGL((sink_window_attention_shared_kernel<DCV, 2 * DCV>), grid, block, 0, stream, a); \
    else hipLaunchKernelGGL((sink_window_attention_grouped_kernel<DCV, 2 * DCV>), grid, block, 0, stream, a);            \
    return;
  if (D > 128) {
    switch (D / 32) { LLMLAB_MFMA_SQUARE(5) LLMLAB_MFMA_SQUARE(6) LLMLAB_MFMA_SQUARE(7) LLMLAB_MFMA_SQUARE(8) }
    return;
  }
#undef LLMLAB_MFMA_SQUARE
  switch (D / 32) {
    case 1: launch_mfma<1>(E / 16, which, grid, block, stream, a); break;
    case 2: launch_mfma<2>(E / 16, which, grid, block, stream, a); break;
    case 3: launch_mfma<3>(E / 16, which, grid, block, stream, a); break;
    default: launch_mfma<4>(E / 16, which, grid, block, stream, a); break;
  }
}

// q [rows, heads * D], out [rows, heads * E] in the compute dtype; sink: float32 [heads] or null.
// The rows of a request are adjacent and requests come in rising order of row_req.
// long_from > 0 (sizes that the matrix-core kernels take only): requests that bring at least so
// many rows (q_start[b + 1] - q_start[b]) go to the prompts' kernel, the others to the decoding
// one; `launches` says which of the two the step needs (bit 0 decoding, bit 1 prompts).
// max_keys: the most keys a decoding row of this step sees (it sets how many shares a row's
// keys are cut into); workspace: float32 scratch for the shares' partial results.
extern "C" int llmlab_sink_window_attention(const void* q, int dtype, int rows, int n_heads, int n_kv, int D, int E,
                                            const void* k_cache, const void* v_cache, const int* table, int max_pages,
                                            int page_size, const int* positions, const int* row_req, int window,
                                            int keep_first, const float* sink, float scale, void* out,
                                            const int* q_start, int long_from, int launches, int max_keys,
                                            float* workspace, size_t workspace_floats, int num_cus, int mode,
                                            hipStream_t stream) {
  LLMLAB_REQUIRE(mode == MODE_SOFTMAX || mode == MODE_SIGMOID, "sink_window_attention: unknown weighting %d", mode);
  LLMLAB_REQUIRE(rows >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0 && D > 0 && E > 0,
                 "sink_window_attention: bad sizes rows=%d heads=%d kv=%d D=%d E=%d", rows, n_heads, n_kv, D, E);
  LLMLAB_REQUIRE(E <= 64 * MAX_E_PER_LANE, "sink_window_attention: values up to %d wide, got %d", 64 * MAX_E_PER_LANE, E);
  LLMLAB_REQUIRE(D <= 4096 && n_heads <= 65535, "sink_window_attention: keys up to 4096 wide and 65535 heads");
  LLMLAB_REQUIRE(keep_first >= 0 && page_size > 0 && page_size % 4 == 0 && max_pages > 0,
                 "sink_window_attention: bad window or page arguments");
  if (rows == 0) return 0;
  if (long_from > 0) {
    LLMLAB_REQUIRE(q_start != nullptr && llmlab_sink_window_attention_has_mfma(dtype, D, E, page_size) && (launches & 3),
                   "sink_window_attention: the matrix-core kernel does not take these sizes (D=%d E=%d page=%d)", D, E,
                   page_size);
  }
  if (long_from > 0) {
    MfmaArgs a{(const bf16_t*)q, rows, n_heads, n_kv, (const bf16_t*)k_cache, (const bf16_t*)v_cache, table, max_pages,
               page_size, positions, row_req, window, keep_first, sink, scale, (bf16_t*)out, q_start, long_from, 1,
               nullptr, nullptr, mode};
    if (launches & 2) {
      // heads that read the same keys and values share the tiles a block stages in LDS
      const int group = n_heads / n_kv;
      if (!g_private_tiles && group >= 3 && (n_kv == 1 || group % 4 == 0))
        launch_mfma_any(D, E, 2, dim3((rows + 15) / 16, (n_heads + 3) / 4), dim3(256), stream, a);
      else
        launch_mfma_any(D, E, 0, dim3((rows + 63) / 64, n_heads), dim3(256), stream, a);
      LLMLAB_LAUNCH_CHECK("sink_window_attention (prompts)");
    }
    if (launches & 1) {
      // shares of a row's keys: enough waves for every compute unit a few times, a share no
      // shorter than two tiles of 32 keys, and no more than the scratch holds
      const int group = n_heads / n_kv, per_group = (group + 15) / 16;
      const long waves = (long)rows * n_kv * per_group;
      const int tiles = (max_keys + 31) / 32 + 1;
      long splits = (4L * num_cus + waves - 1) / waves;
      if (splits > tiles / 2) splits = tiles / 2;
      const size_t per_split = (size_t)rows * n_heads * (E + 2);
      if (workspace == nullptr) splits = 1;
      else if (splits * per_split > workspace_floats) splits = (long)(workspace_floats / per_split);
      if (splits < 1) splits = 1;
      if (splits > MERGE_MAX_SPLITS) splits = MERGE_MAX_SPLITS;
      a.splits = (int)splits;
      a.part_o = workspace;
      a.part_ml = workspace ? workspace + (size_t)rows * n_heads * splits * E : nullptr;
      LLMLAB_REQUIRE(n_kv * per_group <= 65535, "sink_window_attention: too many heads");
      launch_mfma_any(D, E, 1, dim3(rows, n_kv * per_group, a.splits), dim3(64), stream, a);
      LLMLAB_LAUNCH_CHECK("sink_window_attention (decoding)");
      if (a.splits > 1) {
        hipLaunchKernelGGL(sink_window_attention_merge_kernel, dim3(rows, n_heads), dim3(64), 0, stream, a, E);
        LLMLAB_LAUNCH_CHECK("sink_window_attention (merge)");
      }
    }
    return 0;
  }
  const size_t lds = (size_t)(D + 64 + (D & 1)) * sizeof(float) + 64 * sizeof(size_t);
  dim3 grid(rows, n_heads), block(64);
  if (dtype == DT_BF16)
    hipLaunchKernelGGL(sink_window_attention_kernel<bf16_t>, grid, block, lds, stream, (const bf16_t*)q, n_heads, n_kv, D,
                       E, (const bf16_t*)k_cache, (const bf16_t*)v_cache, table, max_pages, page_size, positions,
                       row_req, window, keep_first, sink, scale, (bf16_t*)out, q_start, long_from, mode);
  else
    hipLaunchKernelGGL(sink_window_attention_kernel<float>, grid, block, lds, stream, (const float*)q, n_heads, n_kv, D,
                       E, (const float*)k_cache, (const float*)v_cache, table, max_pages, page_size, positions,
                       row_req, window, keep_first, sink, scale, (float*)out, q_start, long_from, mode);
  LLMLAB_LAUNCH_CHECK("sink_window_attention");
  return 0;
}

// ------------------------------------------------------------------ latent form
// Attention over ONE cached vector per token (kv heads = 1, D = E = the vector's laid-out width,
// the value pages holding the same vector in the values' order): every query head brings its
// query in the vector's coordinates and gets a weighted sum of the vectors back.  The two
// kernels below are what lies around the attention kernels in that form.
//
// One block a row.  proj[r, :] holds float32 projections [q latent (q_laid) | cached latent
// (latent) | gates]: the query's latent is divided by the root mean square over its first
// q_rank numbers and multiplied by q_w; the cached latent likewise (kv_rank, c_w) and written to
// the row's place in both page tensors; the gates are copied as they are.  Numbers behind q_rank
// / kv_rank are padding (zero projections, zero weights).
template <typename T>
__global__ __launch_bounds__(256) void latent_norm_write_kernel(
    const float* __restrict__ proj, int ld, int q_rank, int q_laid, int kv_rank, int latent, int gates, float eps,
    const float* __restrict__ q_w, const float* __restrict__ c_w, T* __restrict__ cq_out, float* __restrict__ gate_out,
    T* __restrict__ k_cache, T* __restrict__ v_cache, int page_size, const int* __restrict__ positions,
    const int* __restrict__ row_req, const int* __restrict__ table, int max_pages) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const float* src = proj + (size_t)r * ld;
  float s = 0.f;
  for (int c = threadIdx.x; c < q_rank; c += blockDim.x) s += src[c] * src[c];
  const float inv_q = 1.0f / sqrtf(block_sum(s, red) / (float)q_rank + eps);
  s = 0.f;
  for (int c = threadIdx.x; c < kv_rank; c += blockDim.x) s += src[q_laid + c] * src[q_laid + c];
  const float inv_c = 1.0f / sqrtf(block_sum(s, red) / (float)kv_rank + eps);
  for (int c = threadIdx.x; c < q_laid; c += blockDim.x)
    cq_out[(size_t)r * q_laid + c] = from_float<T>(src[c] * inv_q * q_w[c]);
  for (int c = threadIdx.x; c < gates; c += blockDim.x) gate_out[(size_t)r * gates + c] = src[q_laid + latent + c];
  const int pos = positions[r];
  const int page = table[(size_t)row_req[r] * max_pages + pos / page_size];
  const int slot = pos % page_size;
  const size_t base = (size_t)page * page_size * latent;
  for (int c = threadIdx.x; c < latent; c += blockDim.x) {
    const T v = from_float<T>(src[q_laid + c] * inv_c * c_w[c]);
    k_cache[base + (size_t)slot * latent + c] = v;
    v_cache[base + value_index(slot, c, latent)] = v;
  }
}

extern "C" int llmlab_latent_norm_write(const float* proj, int ld, int rows, int q_rank, int q_laid, int kv_rank,
                                        int latent, int gates, float eps, const float* q_w, const float* c_w,
                                        void* cq_out, float* gate_out, void* k_cache, void* v_cache, int dtype,
                                        int page_size, const int* positions, const int* row_req, const int* table,
                                        int max_pages, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && q_rank > 0 && q_laid >= q_rank && kv_rank > 0 && latent >= kv_rank && gates >= 0 &&
                     page_size > 0 && page_size % 4 == 0,
                 "latent_norm_write: bad sizes rows=%d q=%d/%d kv=%d/%d gates=%d page=%d", rows, q_rank, q_laid, kv_rank,
                 latent, gates, page_size);
  LLMLAB_REQUIRE(ld >= q_laid + latent + gates, "latent_norm_write: rows of %d numbers do not hold %d", ld,
                 q_laid + latent + gates);
  LLMLAB_REQUIRE(q_w && c_w && cq_out && k_cache && v_cache && positions && row_req && table && (gates == 0 || gate_out),
                 "latent_norm_write: a pointer is missing");
  if (rows == 0) return 0;
  if (dtype == DT_BF16)
    hipLaunchKernelGGL(latent_norm_write_kernel<bf16_t>, dim3(rows), dim3(256), 0, stream, proj, ld, q_rank, q_laid,
                       kv_rank, latent, gates, eps, q_w, c_w, (bf16_t*)cq_out, gate_out, (bf16_t*)k_cache,
                       (bf16_t*)v_cache, page_size, positions, row_req, table, max_pages);
  else
    hipLaunchKernelGGL(latent_norm_write_kernel<float>, dim3(rows), dim3(256), 0, stream, proj, ld, q_rank, q_laid,
                       kv_rank, latent, gates, eps, q_w, c_w, (float*)cq_out, gate_out, (float*)k_cache, (float*)v_cache,
                       page_size, positions, row_req, table, max_pages);
  LLMLAB_LAUNCH_CHECK("latent_norm_write");
  return 0;
}

// out[r, a, :] = w[a] x[r, a, :] for a stack of matrices w [heads, N, K] (row-major), x [rows,
// heads * K], out [rows, heads * N]: every head's numbers through that head's own matrix (a
// query into the cached vector's coordinates; a weighted sum of cached vectors to the head's
// values).  Sums in float32.
//
// Plain kernel (any sizes, both dtypes): a block per (row, head), the head's K numbers in LDS.
template <typename T>
__global__ __launch_bounds__(256) void head_products_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                            T* __restrict__ out, int heads, int N, int K,
                                                            const float* __restrict__ gate) {
  extern __shared__ float xs[];
  const int r = blockIdx.x, a = blockIdx.y;
  const float scale = gate ? 1.f / (1.f + __expf(-gate[(size_t)r * heads + a])) : 1.f;
  const T* xr = x + ((size_t)r * heads + a) * K;
  for (int k = threadIdx.x; k < K; k += blockDim.x) xs[k] = to_float(xr[k]);
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int n = wave; n < N; n += nw) {                 // a wave an output: its lanes share the row of w
    const T* wr = w + ((size_t)a * N + n) * K;
    float s = 0.f;
    for (int k = lane; k < K; k += 64) s = fmaf(to_float(wr[k]), xs[k], s);
    s = wave_sum(s);
    if (lane == 0) out[((size_t)r * heads + a) * N + n] = from_float<T>(s * scale);
  }
}

// Matrix-core kernel (bfloat16, K a multiple of 32, N of 16): a wave takes 16 rows of one head
// and up to HP_TILES tiles of 16 outputs; the product is taken transposed, C^T = W x^T, so that
// a lane ends up with four consecutive outputs of one row (one 8-byte store).
constexpr int HP_TILES = 4;

__global__ __launch_bounds__(256) void head_products_mfma_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                 bf16_t* __restrict__ out, int rows, int heads, int N,
                                                                 int K, const float* __restrict__ gate) {
  const int lane = threadIdx.x & 63, c = lane & 15, g4 = lane >> 4, wave = threadIdx.x >> 6;
  const int r0 = blockIdx.x * 16, a = blockIdx.y;
  const int n_first = (blockIdx.z * 4 + wave) * HP_TILES * 16;
  if (n_first >= N) return;
  const int r = r0 + c;
  const bool row_ok = r < rows;
  const bf16_t* xr = x + ((size_t)(row_ok ? r : rows - 1) * heads + a) * K + 8 * g4;
  const bf16_t* wa = w + (size_t)a * N * K;
  const float gv = gate ? gate[(size_t)(row_ok ? r : rows - 1) * heads + a] : 0.f;
  floatx4 acc[HP_TILES];
  const bf16_t* wr[HP_TILES];
#pragma unroll
  for (int t = 0; t < HP_TILES; ++t) {
    acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
    const int n = n_first + 16 * t + c;
    wr[t] = wa + (size_t)(n < N ? n : N - 1) * K + 8 * g4;       // (a tile past N is computed and not stored)
  }
  for (int k = 0; k < K; k += 32) {
    const bf16x8 xf = *(const bf16x8*)(xr + k);
#pragma unroll
    for (int t = 0; t < HP_TILES; ++t) {
      const bf16x8 wf = *(const bf16x8*)(wr[t] + k);
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, xf, acc[t], 0, 0, 0);
    }
  }
  if (!row_ok) return;
  const float scale = gate ? 1.f / (1.f + __expf(-gv)) : 1.f;
#pragma unroll
  for (int t = 0; t < HP_TILES; ++t) {
    const int n = n_first + 16 * t + 4 * g4;
    if (n >= N) continue;
    bf16x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = (bf16_t)(acc[t][i] * scale);
    *(bf16x4*)(out + ((size_t)r * heads + a) * N + n) = o;
  }
}

// gate: float32 [rows, heads] or null; head a of row r is multiplied by sigmoid(gate[r, a]) before
// the one rounding.
extern "C" int llmlab_head_products(const void* x, const void* w, void* out, int dtype, int rows, int heads, int N,
                                    int K, const float* gate, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && heads > 0 && heads <= 65535 && N > 0 && K > 0 && K <= 12288,
                 "head_products: bad sizes rows=%d heads=%d N=%d K=%d", rows, heads, N, K);
  if (rows == 0) return 0;
  if (dtype == DT_BF16 && !g_force_plain && K % 32 == 0 && N % 16 == 0 && (((uintptr_t)x | (uintptr_t)w) & 15) == 0 &&
      ((uintptr_t)out & 7) == 0) {
    dim3 grid((rows + 15) / 16, heads, (N + 4 * HP_TILES * 16 - 1) / (4 * HP_TILES * 16));
    hipLaunchKernelGGL(head_products_mfma_kernel, grid, dim3(256), 0, stream, (const bf16_t*)x, (const bf16_t*)w,
                       (bf16_t*)out, rows, heads, N, K, gate);
  } else if (dtype == DT_BF16) {
    hipLaunchKernelGGL(head_products_kernel<bf16_t>, dim3(rows, heads), dim3(256), K * sizeof(float), stream,
                       (const bf16_t*)x, (const bf16_t*)w, (bf16_t*)out, heads, N, K, gate);
  } else {
    hipLaunchKernelGGL(head_products_kernel<float>, dim3(rows, heads), dim3(256), K * sizeof(float), stream,
                       (const float*)x, (const float*)w, (float*)out, heads, N, K, gate);
  }
  LLMLAB_LAUNCH_CHECK("head_products");
  return 0;
}
