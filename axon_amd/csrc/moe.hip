// Routing for a mixture of experts: the `top` largest of a token's router logits, their softmax,
// and the (token, chosen expert) pairs listed expert by expert in tiles of up to 16 rows, which
// the grouped product takes as its work list.  Everything stays on the device: the launches of a
// step depend on the number of tokens alone.
#include "api.h"
#include "common.h"

namespace {

// One thread per token.  The largest logit first; of equal logits the lower expert.  Weights:
// exp(z - z_first) over the sum of these, added in the order chosen.
__global__ void route_topk_kernel(const float* __restrict__ logits, int n_tokens, int n_experts, int top,
                                  int32_t* __restrict__ experts, float* __restrict__ weights) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n_tokens) return;
  const float* z = logits + (long)t * n_experts;
  int32_t* chosen = experts + (long)t * top;
  float* w = weights + (long)t * top;
  float first = 0.0f, sum = 0.0f;
  for (int k = 0; k < top; ++k) {
    int best = -1;
    float best_z = 0.0f;
    for (int e = 0; e < n_experts; ++e) {
      bool taken = false;
      for (int j = 0; j < k; ++j) taken |= chosen[j] == e;
      if (taken) continue;
      const float v = z[e];
      if (best < 0 || v > best_z) { best = e; best_z = v; }
    }
    chosen[k] = best;
    if (k == 0) first = best_z;
    const float p = expf(best_z - first);
    w[k] = p;
    sum += p;
  }
  for (int k = 0; k < top; ++k) w[k] = w[k] / sum;
}

// The same choice by a wave per token (up to 1,024 experts: lane l holds the logits of experts l, l + 64, ...):
// `top` times the largest logit not yet taken, by a butterfly over (logit, lower expert first).
__global__ void route_topk_wave_kernel(const float* __restrict__ logits, int n_tokens, int n_experts, int top,
                                       int32_t* __restrict__ experts, float* __restrict__ weights) {
  const int t = blockIdx.x * (blockDim.x / 64) + threadIdx.x / 64, lane = threadIdx.x & 63;
  if (t >= n_tokens) return;
  float z[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) z[i] = lane + 64 * i < n_experts ? logits[(long)t * n_experts + lane + 64 * i] : -INFINITY;
  unsigned taken = 0;
  float first = 0.0f, sum = 0.0f, mine = 0.0f;        // lane k keeps the k-th weight
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int e = lane + 64 * i;
      if (e < n_experts && !(taken >> i & 1) && (at == 0x7fffffff || z[i] > best)) { best = z[i]; at = e; }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float other = __shfl_xor(best, off, 64);
      const int other_at = __shfl_xor(at, off, 64);
      if (other_at != 0x7fffffff && (at == 0x7fffffff || other > best || (other == best && other_at < at))) { best = other; at = other_at; }
    }
    if ((at & 63) == lane) taken |= 1u << (at >> 6);
    if (k == 0) first = best;
    const float p = expf(best - first);
    sum += p;
    if (lane == k % 64) { mine = p; experts[(long)t * top + k] = at; }
  }
  if (lane < top) weights[(long)t * top + lane] = mine / sum;
}

// Scores that do not compete: s_e = sigmoid(z_e); the choice is made by s_e + correction_e (if given),
// the weights come from s_e alone.  The experts form `groups` equal groups of neighbours; a group's
// score is the sum of its two largest choice scores (of its one, if it has one expert), only experts
// of the `keep` best groups can be chosen (of equal groups the lower), and among those the `top`
// largest choice scores win (of equal ones the lower expert).  weights_k = s_k / (sum of the chosen s,
// added in the order chosen, + 1e-20) * scale, or without `normalize` the score itself times scale.  Rows of
// logits are logits_stride apart (further columns may hold other products of the same input).  A wave per token: lane l holds experts l, l + 64, ...
// (up to 1,024) and, for the groups' scores, walks group l (up to 64 groups).
__global__ void route_scored_wave_kernel(const float* __restrict__ logits, long logits_stride, const float* __restrict__ correction,
                                         int n_tokens, int n_experts, int top, int groups, int keep, float scale, int normalize,
                                         int32_t* __restrict__ experts, float* __restrict__ weights) {
  const int t = blockIdx.x * (blockDim.x / 64) + threadIdx.x / 64, lane = threadIdx.x & 63;
  if (t >= n_tokens) return;
  const float* z = logits + (long)t * logits_stride;
  const int size = n_experts / groups;
  unsigned long long kept = ~0ull;
  if (groups > 1) {
    float first = -INFINITY, second = -INFINITY;
    if (lane < groups)
      for (int e = lane * size; e < (lane + 1) * size; ++e) {
        const float c = 1.0f / (1.0f + expf(-z[e])) + (correction ? correction[e] : 0.0f);
        if (c > first) { second = first; first = c; }
        else if (c > second) second = c;
      }
    const float mine = size > 1 ? first + second : first;
    int ahead = 0;                                   // groups that rank before this lane's
    for (int g = 0; g < groups; ++g) {
      const float other = __shfl(mine, g, 64);
      ahead += (other > mine || (other == mine && g < lane)) ? 1 : 0;
    }
    kept = __ballot(lane < groups && ahead < keep);
  }
  float choice[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int e = lane + 64 * i;
    choice[i] = -INFINITY;
    if (e < n_experts && (kept >> (e / size) & 1)) choice[i] = 1.0f / (1.0f + expf(-z[e])) + (correction ? correction[e] : 0.0f);
  }
  unsigned taken = 0;
  float sum = 0.0f, mine = 0.0f;                     // lane k keeps the k-th score
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int e = lane + 64 * i;
      if (e < n_experts && (kept >> (e / size) & 1) && !(taken >> i & 1) && (at == 0x7fffffff || choice[i] > best)) { best = choice[i]; at = e; }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float other = __shfl_xor(best, off, 64);
      const int other_at = __shfl_xor(at, off, 64);
      if (other_at != 0x7fffffff && (at == 0x7fffffff || other > best || (other == best && other_at < at))) { best = other; at = other_at; }
    }
    if ((at & 63) == lane) taken |= 1u << (at >> 6);
    const float s = 1.0f / (1.0f + expf(-z[at]));
    sum += s;
    if (lane == k % 64) { mine = s; experts[(long)t * top + k] = at; }
  }
  if (lane < top) weights[(long)t * top + lane] = normalize ? (mine / (sum + 1e-20f)) * scale : mine * scale;
}

// One block.  pairs p = t top + k in expert order -> sorted [n_pairs], with the token of each
// (sorted_tokens); tiles [.][3] = (expert, first place in sorted, count <= tile_rows), *n_tiles of them.
// Which place a pair gets inside its expert's stretch is not fixed (atomic counters); no result
// depends on it: every row of a product is a chain of its own.
__global__ void __launch_bounds__(1024)
route_sort_kernel(const int32_t* __restrict__ experts, int n_pairs, int n_experts, int top, int32_t* __restrict__ sorted,
                  int32_t* __restrict__ sorted_tokens, int32_t* __restrict__ tiles, int32_t* __restrict__ n_tiles,
                  int32_t* __restrict__ place_of, int32_t* __restrict__ first_of, int tile_rows) {
  extern __shared__ int counts[];              // [n_experts] counts, then [n_experts] next free places
  int* next = counts + n_experts;
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) atomicAdd(&counts[experts[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, tile = 0;
    for (int e = 0; e < n_experts; ++e) {
      const int n = counts[e];
      next[e] = at;
      if (first_of) first_of[e] = at;
      for (int i = 0; i < n; i += tile_rows) {
        tiles[3 * tile] = e; tiles[3 * tile + 1] = at + i; tiles[3 * tile + 2] = min(tile_rows, n - i);
        ++tile;
      }
      at += n;
    }
    *n_tiles = tile;
    if (first_of) first_of[n_experts] = at;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) {
    const int place = atomicAdd(&next[experts[p]], 1);
    sorted[place] = p;
    sorted_tokens[place] = p / top;
    if (place_of) place_of[p] = place;
  }
}

// y[t, :] (+)= sum_k weights[t, k] rows[row of pair t top + k, :], k ascending; a pair's row is the pair
// itself, or place_of[pair]; without weights the rows are added as they are.  extra (or null): a further
// row a token, added last, times sigmoid(extra_gate[t extra_gate_stride]) if a gate is given.
__global__ void route_combine_kernel(const float* __restrict__ rows, const float* __restrict__ weights, float* __restrict__ y,
                                     int top, int width, int accumulate, const int32_t* __restrict__ place_of,
                                     const float* __restrict__ extra, const float* __restrict__ extra_gate, long extra_gate_stride) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= width) return;
  float acc = accumulate ? y[(long)t * width + c] : 0.0f;
  for (int k = 0; k < top; ++k) {
    const long pair = (long)t * top + k;
    const float row = rows[(place_of ? (long)place_of[pair] : pair) * width + c];
    acc = weights ? fmaf(weights[pair], row, acc) : acc + row;
  }
  if (extra) {
    const float e = extra[(long)t * width + c];
    acc = extra_gate ? fmaf(1.0f / (1.0f + expf(-extra_gate[(long)t * extra_gate_stride])), e, acc) : acc + e;
  }
  y[(long)t * width + c] = acc;
}

// out[r, :] = x[rows[r], :] (rows of the compute dtype).
__global__ void gather_rows_kernel(const elem_t* __restrict__ x, long x_stride, const int32_t* __restrict__ rows,
                                   elem_t* __restrict__ out, int width) {
  const elem_t* src = x + (long)rows[blockIdx.x] * x_stride;
  elem_t* dst = out + (long)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = src[i];
}

}  // namespace

extern "C" int axk_route_topk(const float* logits, int n_tokens, int n_experts, int top, int32_t* experts, float* weights,
                              void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && n_experts > 0 && top > 0 && top <= n_experts, "route_topk: %d tokens, %d of %d experts",
              n_tokens, top, n_experts);
  if (n_tokens == 0) return 0;
  if (n_experts <= 1024 && top <= 64) {
    route_topk_wave_kernel<<<ceil_div(n_tokens, 4), 256, 0, (hipStream_t)stream>>>(logits, n_tokens, n_experts, top, experts, weights);
    AXK_LAUNCH_CHECK("route_topk");
    return 0;
  }
  route_topk_kernel<<<ceil_div(n_tokens, 64), 64, 0, (hipStream_t)stream>>>(logits, n_tokens, n_experts, top, experts, weights);
  AXK_LAUNCH_CHECK("route_topk");
  return 0;
}

extern "C" int axk_route_scored(const float* logits, long logits_stride, const float* correction, int n_tokens, int n_experts,
                                int top, int groups, int keep, float scale, int normalize, int32_t* experts, float* weights,
                                void* stream) {
  AXK_REQUIRE(logits_stride >= n_experts, "route_scored: rows of %ld logits for %d experts", logits_stride, n_experts);
  AXK_REQUIRE(n_tokens >= 0 && n_experts > 0 && n_experts <= 1024 && top > 0 && top <= 64,
              "route_scored: %d tokens, %d of %d experts (at most 64 of 1024)", n_tokens, top, n_experts);
  AXK_REQUIRE(groups >= 1 && groups <= 64 && n_experts % groups == 0 && keep >= 1 && keep <= groups &&
              (long)keep * (n_experts / groups) >= top,
              "route_scored: %d of %d groups of %d experts for %d a token", keep, groups, n_experts / (groups > 0 ? groups : 1), top);
  if (n_tokens == 0) return 0;
  route_scored_wave_kernel<<<ceil_div(n_tokens, 4), 256, 0, (hipStream_t)stream>>>(logits, logits_stride, correction, n_tokens, n_experts, top,
                                                                                  groups, keep, scale, normalize, experts, weights);
  AXK_LAUNCH_CHECK("route_scored");
  return 0;
}

extern "C" int axk_route_max_tiles(int n_pairs, int n_experts, int tile_rows) {
  return ceil_div(n_pairs, tile_rows > 0 ? tile_rows : 16) + n_experts;
}

extern "C" int axk_gather_rows(const void* x, long x_stride, const int32_t* rows, void* out, int n_rows, int width, void* stream) {
  AXK_REQUIRE(n_rows >= 0 && width > 0 && x_stride >= width, "gather_rows: %d rows of %d (stride %ld)", n_rows, width, x_stride);
  if (n_rows == 0) return 0;
  gather_rows_kernel<<<n_rows, 256, 0, (hipStream_t)stream>>>((const elem_t*)x, x_stride, rows, (elem_t*)out, width);
  AXK_LAUNCH_CHECK("gather_rows");
  return 0;
}

extern "C" int axk_route_sort(const int32_t* experts, int n_pairs, int n_experts, int top, int32_t* sorted,
                              int32_t* sorted_tokens, int32_t* tiles, int32_t* n_tiles, int32_t* place_of, int32_t* first_of,
                              int tile_rows, void* stream) {
  AXK_REQUIRE(n_pairs >= 0 && n_experts > 0 && top > 0 && n_experts <= 4096 && tile_rows > 0,
              "route_sort: %d pairs, %d experts, tiles of %d", n_pairs, n_experts, tile_rows);
  route_sort_kernel<<<1, 1024, 2 * n_experts * sizeof(int), (hipStream_t)stream>>>(experts, n_pairs, n_experts, top, sorted,
                                                                                  sorted_tokens, tiles, n_tiles, place_of, first_of, tile_rows);
  AXK_LAUNCH_CHECK("route_sort");
  return 0;
}

extern "C" int axk_route_combine(const float* rows, const float* weights, float* y, int n_tokens, int top, int width,
                                 int accumulate, const int32_t* place_of, const float* extra, const float* extra_gate,
                                 long extra_gate_stride, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && top > 0 && width > 0 && n_tokens <= 65535, "route_combine: T=%d top=%d width=%d", n_tokens, top,
              width);
  if (n_tokens == 0) return 0;
  dim3 grid(ceil_div(width, 256), n_tokens);
  route_combine_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(rows, weights, y, top, width, accumulate, place_of, extra,
                                                              extra_gate, extra_gate_stride);
  AXK_LAUNCH_CHECK("route_combine");
  return 0;
}
