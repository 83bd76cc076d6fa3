// A feed-forward made of many small ones (experts) of which every row uses a few: the choice,
// the sorting of rows by expert, and the sum of the chosen experts' results, for gfx950.
//
//   select      per row: softmax over the router's outputs, choice value = score + correction,
//               the best groups of neighbours, the top outputs among them; weight = score * scale
//   add_chosen  resid[r] += (sum of the weights of row r's choices within [first, last)) * src[r]
#include "common.h"

extern "C" const char* llmlab_last_error() { return g_llmlab_error; }

constexpr int SELECT_MAX_OUTPUTS = 1024;     // router outputs a row's wave keeps in LDS

// One wave a row.  Everything in float32; ties go to the smaller index, as a scan in order does.
__global__ __launch_bounds__(64) void moe_select_kernel(const float* __restrict__ logits, const float* __restrict__ correction,
                                                        int outputs, int groups, int keep, int top, float scale,
                                                        int* __restrict__ chosen, float* __restrict__ weights,
                                                        int sigmoid) {
  __shared__ float s_score[SELECT_MAX_OUTPUTS], s_choice[SELECT_MAX_OUTPUTS];
  __shared__ float s_group[SELECT_MAX_OUTPUTS];
  const int row = blockIdx.x, lane = threadIdx.x;
  const float* z = logits + (size_t)row * outputs;
  float m = -INFINITY;
  for (int e = lane; e < outputs; e += WAVE) m = fmaxf(m, z[e]);
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
  float sum = 0.f;
  for (int e = lane; e < outputs; e += WAVE) {
    const float p = sigmoid ? 1.f / (1.f + expf(-z[e])) : expf(z[e] - m);
    s_score[e] = p;
    sum += p;
  }
  for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
  const float inv = sigmoid ? 1.f : 1.f / sum;          // (sigmoid: every output scores by itself)
  for (int e = lane; e < outputs; e += WAVE) {
    const float s = s_score[e] * inv;
    s_score[e] = s;
    s_choice[e] = s + correction[e];
  }
  __syncthreads();
  const int per = outputs / groups;
  if (keep < groups) {
    for (int g = lane; g < groups; g += WAVE) {
      float best = -INFINITY;
      for (int i = 0; i < per; ++i) best = fmaxf(best, s_choice[g * per + i]);
      s_group[g] = best;
    }
    __syncthreads();
    // a group is kept if fewer than `keep` groups come before it in the order (value down, index up)
    for (int g = lane; g < groups; g += WAVE) {
      const float mine = s_group[g];
      int before = 0;
      for (int o = 0; o < groups; ++o) {
        const float other = s_group[o];
        before += (other > mine) || (other == mine && o < g);
      }
      if (before >= keep)
        for (int i = 0; i < per; ++i) s_choice[g * per + i] = -INFINITY;
    }
    __syncthreads();
  }
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = outputs;             // (when every value left is minus infinity: the smallest index left)
    for (int e = lane; e < outputs; e += WAVE) {
      const float c = s_choice[e];
      if (c > best || (c == best && e < at)) {
        best = c;
        at = e;
      }
    }
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o);
      const int oa = __shfl_xor(at, o);
      if (ob > best || (ob == best && oa < at)) {
        best = ob;
        at = oa;
      }
    }
    at = min(at, outputs - 1);
    if (lane == 0) {
      chosen[(size_t)row * top + k] = at;
      weights[(size_t)row * top + k] = s_score[at] * scale;
      s_choice[at] = -INFINITY;          // taken
    }
    __syncthreads();
  }
}

// The same for a router of up to 64 outputs: a lane an output, a wave a row, no block barrier.
// A lane finds its place in the order (value down, index up) by reading every output's value
// from the wave's own 64 floats of LDS: reads of one address by all lanes, independent of each
// other, so they pipeline.  (A chain of lane-to-lane exchanges per chosen output, six steps of a
// reduction each, cost 8 to 11 us for 8 rows; reads of another lane's register in a loop over
// the outputs were no faster.)
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ __forceinline__ void select_row_by_wave(const float* __restrict__ logits, const float* __restrict__ correction,
                                                   int outputs, int groups, int keep, int top, float scale,
                                                   int* __restrict__ chosen, float* __restrict__ weights, int row,
                                                   int lane, float* s_wave, int sigmoid) {
  const bool mine = lane < outputs;
  const float z = mine ? logits[(size_t)row * outputs + lane] : -INFINITY;
  wave_sync();                                 // (the row before is read out)
  s_wave[lane] = z;
  wave_sync();
  float m = -INFINITY;
  for (int j = 0; j < outputs; ++j) m = fmaxf(m, s_wave[j]);
  const float p = mine ? (sigmoid ? 1.f / (1.f + expf(-z)) : expf(z - m)) : 0.f;
  s_wave[WAVE + lane] = p;
  wave_sync();
  float sum = 0.f;
  for (int j = 0; j < outputs; ++j) sum += s_wave[WAVE + j];         // (in the order of the outputs, on every lane)
  const float score = sigmoid ? p : p * (1.f / sum);
  float choice = mine ? score + correction[lane] : -INFINITY;
  wave_sync();
  s_wave[lane] = choice;
  wave_sync();
  if (keep < groups) {
    const int per = outputs / groups, g = mine ? lane / per : groups;
    float best = -INFINITY;                    // of this lane's group
    if (mine)
      for (int i = 0; i < per; ++i) best = fmaxf(best, s_wave[g * per + i]);
    wave_sync();
    s_wave[WAVE + lane] = best;
    wave_sync();
    int before = 0;                            // groups that come before this lane's
    for (int o = 0; o < groups; ++o) {
      const float other = s_wave[WAVE + o * per];
      before += (other > best) || (other == best && o < g);
    }
    if (before >= keep) choice = -INFINITY;
    wave_sync();
    s_wave[lane] = choice;
    wave_sync();
  }
  int place = 0;                               // outputs that come before this lane's
  for (int j = 0; j < outputs; ++j) {
    const float c = s_wave[j];
    place += (c > choice) || (c == choice && j < lane);
  }
  if (mine && place < top) {
    chosen[(size_t)row * top + place] = lane;
    weights[(size_t)row * top + place] = score * scale;
  }
}

__global__ __launch_bounds__(64) void moe_select_wave_kernel(const float* __restrict__ logits,
                                                             const float* __restrict__ correction, int outputs, int groups,
                                                             int keep, int top, float scale, int* __restrict__ chosen,
                                                             float* __restrict__ weights, int sigmoid) {
  __shared__ float s_wave[2 * WAVE];
  select_row_by_wave(logits, correction, outputs, groups, keep, top, scale, chosen, weights, blockIdx.x, threadIdx.x,
                     s_wave, sigmoid);
}

// scoring: 0 softmax over the outputs, 1 the sigmoid of each output by itself
extern "C" int llmlab_moe_select(const float* logits, const float* correction, int rows, int outputs, int groups,
                                 int keep, int top, float scale, int* chosen, float* weights, int scoring,
                                 hipStream_t stream) {
  LLMLAB_REQUIRE(scoring == 0 || scoring == 1, "moe_select: scoring %d", scoring);
  LLMLAB_REQUIRE(rows >= 0 && outputs > 0 && outputs <= SELECT_MAX_OUTPUTS,
                 "moe_select: a router of 1 to %d outputs, got %d", SELECT_MAX_OUTPUTS, outputs);
  LLMLAB_REQUIRE(groups > 0 && outputs % groups == 0 && keep > 0 && keep <= groups && top > 0 &&
                     top <= keep * (outputs / groups),
                 "moe_select: %d outputs in %d groups of which %d are kept, top %d", outputs, groups, keep, top);
  if (rows == 0) return 0;
  if (outputs <= WAVE)
    hipLaunchKernelGGL(moe_select_wave_kernel, dim3(rows), dim3(64), 0, stream, logits, correction, outputs, groups,
                       keep, top, scale, chosen, weights, scoring);
  else
    hipLaunchKernelGGL(moe_select_kernel, dim3(rows), dim3(64), 0, stream, logits, correction, outputs, groups, keep,
                       top, scale, chosen, weights, scoring);
  LLMLAB_LAUNCH_CHECK("moe_select");
  return 0;
}

// resid[r, :] += w_r * src[r, :],  w_r = sum of weights[r, k] over the k with first <= chosen[r, k] < last
template <typename T>
__global__ void moe_add_chosen_kernel(float* __restrict__ resid, const T* __restrict__ src, const int* __restrict__ chosen,
                                      const float* __restrict__ weights, int top, int first, int last, int hidden) {
  const int row = blockIdx.x;
  float w = 0.f;
  bool any = false;
  for (int k = 0; k < top; ++k) {
    const int e = chosen[(size_t)row * top + k];
    if (e >= first && e < last) {
      w += weights[(size_t)row * top + k];
      any = true;
    }
  }
  if (!any) return;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x)
    resid[(size_t)row * hidden + i] += w * to_float(src[(size_t)row * hidden + i]);
}

extern "C" int llmlab_moe_add_chosen(float* resid, const void* src, int src_dtype, const int* chosen,
                                     const float* weights, int rows, int top, int first, int last, int hidden,
                                     hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && top > 0 && hidden > 0, "moe_add_chosen: bad sizes rows=%d top=%d hidden=%d", rows, top,
                 hidden);
  if (rows == 0 || first >= last) return 0;
  if (src_dtype == DT_BF16)
    hipLaunchKernelGGL(moe_add_chosen_kernel<bf16_t>, dim3(rows), dim3(256), 0, stream, resid, (const bf16_t*)src,
                       chosen, weights, top, first, last, hidden);
  else
    hipLaunchKernelGGL(moe_add_chosen_kernel<float>, dim3(rows), dim3(256), 0, stream, resid, (const float*)src, chosen,
                       weights, top, first, last, hidden);
  LLMLAB_LAUNCH_CHECK("moe_add_chosen");
  return 0;
}

// ------------------------------------------------------------------ rows sorted by expert
// The (row, choice) pairs of a step, sorted by expert into tiles of `bm` places that a grouped
// product walks: every expert's pairs are consecutive and start at a multiple of bm.
//   place_of[rows * top]   the place of a pair (-1: the pair chose no expert with tensors)
//   place_row[capacity]    the row of x at a place (-1: the place is padding)
//   tile_member[capacity / bm]   the expert of a tile of places (-1: past the last tile in use)
// capacity = (pairs + experts * (bm - 1)) rounded up to whole tiles, whatever the choice: the
// buffers and the grids that walk them have sizes the host knows.  One block: counts by atomic
// adds in LDS, a scan over the experts, places handed out by atomic adds in LDS.  Which place
// of its expert a pair gets depends on the order of those adds; no result does, because a row
// of a product depends on that row alone.
constexpr int PLAN_MAX_EXPERTS = 1024;

__device__ __forceinline__ void plan_by_block(const int* __restrict__ chosen, int pairs, int experts, int bm, int capacity,
                                              int* __restrict__ place_of, int* __restrict__ place_row,
                                              int* __restrict__ tile_member, int top, int* s_count, int* s_start) {
  const int tid = threadIdx.x, nt = blockDim.x;
  for (int e = tid; e < experts; e += nt) s_count[e] = 0;
  for (int i = tid; i < capacity; i += nt) place_row[i] = -1;
  for (int t = tid; t < capacity / bm; t += nt) tile_member[t] = -1;
  __syncthreads();
  // (four pairs a load where the pairs allow it: a thread's loads are a chain of trips to memory)
  const int quads = (((uintptr_t)chosen | (uintptr_t)place_of) % 16 == 0) ? pairs / 4 : 0;
  for (int q = tid; q < quads; q += nt) {
    const int4 c = ((const int4*)chosen)[q];
    const int e4[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (e4[i] >= 0 && e4[i] < experts) atomicAdd(&s_count[e4[i]], 1);
  }
  for (int p = 4 * quads + tid; p < pairs; p += nt) {
    const int e = chosen[p];
    if (e >= 0 && e < experts) atomicAdd(&s_count[e], 1);
  }
  __syncthreads();
  if (tid == 0) {
    int at = 0;
    for (int e = 0; e < experts; ++e) {
      s_start[e] = at;
      at += (s_count[e] + bm - 1) / bm * bm;
    }
  }
  __syncthreads();
  for (int e = tid; e < experts; e += nt) {
    const int first = s_start[e] / bm, tiles = (s_count[e] + bm - 1) / bm;
    for (int t = 0; t < tiles; ++t) tile_member[first + t] = e;
    s_count[e] = 0;                      // from here on: places handed out
  }
  __syncthreads();
  for (int q = tid; q < quads; q += nt) {
    const int4 c = ((const int4*)chosen)[q];
    const int e4[4] = {c.x, c.y, c.z, c.w};
    int place[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      place[i] = -1;
      if (e4[i] >= 0 && e4[i] < experts) {
        place[i] = s_start[e4[i]] + atomicAdd(&s_count[e4[i]], 1);
        place_row[place[i]] = (4 * q + i) / top;
      }
    }
    ((int4*)place_of)[q] = make_int4(place[0], place[1], place[2], place[3]);
  }
  for (int p = 4 * quads + tid; p < pairs; p += nt) {
    const int e = chosen[p];
    int place = -1;
    if (e >= 0 && e < experts) {
      place = s_start[e] + atomicAdd(&s_count[e], 1);
      place_row[place] = p / top;
    }
    place_of[p] = place;
  }
}

__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* __restrict__ chosen, int pairs, int experts, int bm,
                                                        int capacity, int* __restrict__ place_of,
                                                        int* __restrict__ place_row, int* __restrict__ tile_member,
                                                        int top) {
  __shared__ int s_count[PLAN_MAX_EXPERTS], s_start[PLAN_MAX_EXPERTS];
  plan_by_block(chosen, pairs, experts, bm, capacity, place_of, place_row, tile_member, top, s_count, s_start);
}

// Choice and sorting of a step of few rows in one launch: the waves of the one block take the rows
// in turn, then the block sorts what they chose (their writes are the block's own: a barrier
// makes them seen).
__global__ __launch_bounds__(1024) void moe_select_plan_kernel(const float* __restrict__ logits,
                                                               const float* __restrict__ correction, int rows, int outputs,
                                                               int groups, int keep, int top, float scale,
                                                               int* __restrict__ chosen, float* __restrict__ weights,
                                                               int experts, int bm, int capacity, int* __restrict__ place_of,
                                                               int* __restrict__ place_row, int* __restrict__ tile_member,
                                                               int sigmoid) {
  __shared__ int s_count[PLAN_MAX_EXPERTS], s_start[PLAN_MAX_EXPERTS];
  __shared__ float s_waves[16][2 * WAVE];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, waves = blockDim.x >> 6;
  for (int row = wave; row < rows; row += waves)
    select_row_by_wave(logits, correction, outputs, groups, keep, top, scale, chosen, weights, row, lane, s_waves[wave],
                       sigmoid);
  __threadfence_block();
  __syncthreads();
  plan_by_block(chosen, rows * top, experts, bm, capacity, place_of, place_row, tile_member, top, s_count, s_start);
}

extern "C" int llmlab_moe_select_plan(const float* logits, const float* correction, int rows, int outputs, int groups,
                                      int keep, int top, float scale, int* chosen, float* weights, int experts, int bm,
                                      int capacity, int* place_of, int* place_row, int* tile_member, int scoring,
                                      hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && outputs > 0 && outputs <= WAVE, "moe_select_plan: a router of 1 to 64 outputs, got %d",
                 outputs);
  LLMLAB_REQUIRE(scoring == 0 || scoring == 1, "moe_select_plan: scoring %d", scoring);
  LLMLAB_REQUIRE(groups > 0 && outputs % groups == 0 && keep > 0 && keep <= groups && top > 0 &&
                     top <= keep * (outputs / groups),
                 "moe_select_plan: %d outputs in %d groups of which %d are kept, top %d", outputs, groups, keep, top);
  LLMLAB_REQUIRE(experts > 0 && experts <= PLAN_MAX_EXPERTS && bm > 0, "moe_select_plan: experts=%d bm=%d", experts, bm);
  const long need = ((long)rows * top + (long)experts * (bm - 1) + bm - 1) / bm * bm;
  LLMLAB_REQUIRE(capacity % bm == 0 && capacity >= need, "moe_select_plan: %d places for %d pairs of %d experts", capacity,
                 rows * top, experts);
  if (rows == 0) return 0;
  hipLaunchKernelGGL(moe_select_plan_kernel, dim3(1), dim3(1024), 0, stream, logits, correction, rows, outputs, groups,
                     keep, top, scale, chosen, weights, experts, bm, capacity, place_of, place_row, tile_member, scoring);
  LLMLAB_LAUNCH_CHECK("moe_select_plan");
  return 0;
}

extern "C" int llmlab_moe_plan(const int* chosen, int rows, int top, int experts, int bm, int capacity, int* place_of,
                               int* place_row, int* tile_member, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && top > 0 && experts > 0 && experts <= PLAN_MAX_EXPERTS && bm > 0,
                 "moe_plan: bad sizes rows=%d top=%d experts=%d bm=%d", rows, top, experts, bm);
  const long need = ((long)rows * top + (long)experts * (bm - 1) + bm - 1) / bm * bm;
  LLMLAB_REQUIRE(capacity % bm == 0 && capacity >= need, "moe_plan: %d places for %d pairs of %d experts in tiles of %d",
                 capacity, rows * top, experts, bm);
  if (rows == 0) return 0;
  hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), 0, stream, chosen, rows * top, experts, bm, capacity, place_of,
                     place_row, tile_member, top);
  LLMLAB_LAUNCH_CHECK("moe_plan");
  return 0;
}

// resid[r, :] += sum_k weights[r, k] * (y[place_of[r, k], :]  or, for a choice at or beyond
// `experts` (an identity output), h[r, :]), the choices in their order.  One block a row.
template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ resid, const float* __restrict__ y,
                                                          const T* __restrict__ h, const int* __restrict__ place_of,
                                                          const int* __restrict__ chosen,
                                                          const float* __restrict__ weights, int top, int experts,
                                                          int hidden, const float* __restrict__ extra) {
  const int row = blockIdx.x;
  const int* places = place_of + (size_t)row * top;
  const float* w = weights + (size_t)row * top;
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < hidden; i += gridDim.y * blockDim.x) {
    float sum = 0.f;
    for (int k = 0; k < top; ++k) {
      const int place = places[k];
      if (place >= 0)
        sum += w[k] * y[(size_t)place * hidden + i];
      else if (chosen[(size_t)row * top + k] >= experts)
        sum += w[k] * to_float(h[(size_t)row * hidden + i]);
    }
    resid[(size_t)row * hidden + i] += sum;
  }
}

extern "C" int llmlab_moe_combine(float* resid, const float* y, const void* h, int h_dtype, const int* place_of,
                                  const int* chosen, const float* weights, int rows, int top, int experts, int hidden,
                                  hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && top > 0 && hidden > 0, "moe_combine: bad sizes rows=%d top=%d hidden=%d", rows, top,
                 hidden);
  if (rows == 0) return 0;
  // few rows: the columns of a row are spread over several blocks, so that the chip has work
  const int across = rows >= 1024 ? 1 : min((hidden + 255) / 256, max(1, 1024 / rows));
  const dim3 grid(rows, across);
  if (h_dtype == DT_BF16)
    hipLaunchKernelGGL(moe_combine_kernel<bf16_t>, grid, dim3(256), 0, stream, resid, y, (const bf16_t*)h, place_of,
                       chosen, weights, top, experts, hidden, (const float*)nullptr);
  else
    hipLaunchKernelGGL(moe_combine_kernel<float>, grid, dim3(256), 0, stream, resid, y, (const float*)h, place_of,
                       chosen, weights, top, experts, hidden, (const float*)nullptr);
  LLMLAB_LAUNCH_CHECK("moe_combine");
  return 0;
}
