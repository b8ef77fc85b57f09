// Row-wise kernels: embedding gather, RMSNorm, rotary tables, rotary + paged cache store,
// SwiGLU, fills.  Each computes a row the same way whatever other rows share the launch.
#include "api.h"
#include "common.h"
#include "instances.h"

// ---------------------------------------------------------------------------- embedding
// One block per token; the row is widened exactly (bf16 -> f32) or copied.
// Reference twin: embed_b (src/cuda/prefill.cu:52-56); no scaling for this architecture
// (src/model.rs:2657-2675).
// A tied head's matrix is kept packed for the products (see axk_pack_matrix): element (row, i) is
// then at ((row / 16 * dim / 32 + i / 32) * 64 + row % 16 + 16 (i % 32 / 8)) * 8 + i % 8.
__global__ void embed_kernel(const int32_t* __restrict__ tokens, const elem_t* __restrict__ table, int packed,
                             float* __restrict__ x, int dim, float scale) {
  const int t = blockIdx.x;
  const int token = tokens[t];
  float* dst = x + (size_t)t * dim;
  if (packed) {
    const elem_t* tile = table + (size_t)(token / 16) * (dim / 32) * 512 + (token % 16) * 8;
    for (int i = threadIdx.x; i < dim; i += blockDim.x)
      dst[i] = to_float(tile[(size_t)(i / 32) * 512 + ((i % 32) / 8) * 128 + i % 8]) * scale;
    return;
  }
  const elem_t* row = table + (size_t)token * dim;
  for (int i = threadIdx.x; i < dim; i += blockDim.x) dst[i] = to_float(row[i]) * scale;
}

extern "C" int axk_embed_scaled(const int32_t* tokens, const void* table, int packed, float* x, int n_tokens, int dim,
                                int vocab, float scale, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && dim > 0 && vocab > 0, "embed: bad sizes T=%d dim=%d vocab=%d", n_tokens, dim, vocab);
  AXK_REQUIRE(!packed || dim % 32 == 0, "embed: a packed table has rows of whole blocks of 32, not %d", dim);
  if (n_tokens == 0) return 0;
  embed_kernel<<<n_tokens, 256, 0, (hipStream_t)stream>>>(tokens, (const elem_t*)table, packed, x, dim, scale);
  AXK_LAUNCH_CHECK("embed");
  return 0;
}

// a factor of 1 leaves the widened values as they are
extern "C" int axk_embed(const int32_t* tokens, const void* table, int packed, float* x, int n_tokens, int dim,
                         int vocab, void* stream) {
  return axk_embed_scaled(tokens, table, packed, x, n_tokens, dim, vocab, 1.0f, stream);
}

// ---------------------------------------------------------------------------- RMSNorm
// ss = sum x^2 (32-bit), ms = ss / n, inv = 1 / sqrt(ms + eps), out = (x * inv) * g: x times
// inv first, then the gain (src/model.rs:3888-3898).  The sum is a strided chain per thread,
// a butterfly per wave and the four waves in order: fixed by `dim` alone
// (the reference's GPU twin does the same: src/cuda/decode.cu:212-249).
#define NORM_THREADS 256
#define NORM_CACHED 4  // float4 a thread keeps in registers: rows up to 4096 wide are read once

__device__ inline void store4(elem_t* dst, float a, float b, float c, float d) {
#if AXON_BF16
  uint2 pk;
  pk.x = (uint32_t)float_to_bf16(a).bits | ((uint32_t)float_to_bf16(b).bits << 16);
  pk.y = (uint32_t)float_to_bf16(c).bits | ((uint32_t)float_to_bf16(d).bits << 16);
  *reinterpret_cast<uint2*>(dst) = pk;
#else
  *reinterpret_cast<float4*>(dst) = make_float4(a, b, c, d);
#endif
}

// Rows whose width is a multiple of 4: thread t takes the float4 t, t + 256, ...; the first
// NORM_CACHED of them stay in registers between the sum and the scaling.  The order of the
// sum depends on the width alone.
__global__ void __launch_bounds__(NORM_THREADS)
rmsnorm_vec_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows, const void* __restrict__ gain,
                   int gain_is_f32, elem_t* __restrict__ out, int dim, float eps) {
  __shared__ float partial[NORM_THREADS / AXON_WAVE];
  const int r = blockIdx.x, n4 = dim >> 2;
  const float4* src = reinterpret_cast<const float4*>(x + (size_t)(rows ? rows[r] : r) * dim);
  float4 kept[NORM_CACHED];
  float ss = 0.0f;
#pragma unroll
  for (int c = 0; c < NORM_CACHED; ++c) {
    const int i = threadIdx.x + c * NORM_THREADS;
    kept[c] = i < n4 ? src[i] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    ss = fmaf(kept[c].x, kept[c].x, ss);
    ss = fmaf(kept[c].y, kept[c].y, ss);
    ss = fmaf(kept[c].z, kept[c].z, ss);
    ss = fmaf(kept[c].w, kept[c].w, ss);
  }
  for (int i = threadIdx.x + NORM_CACHED * NORM_THREADS; i < n4; i += NORM_THREADS) {
    const float4 v = src[i];
    ss = fmaf(v.x, v.x, ss);
    ss = fmaf(v.y, v.y, ss);
    ss = fmaf(v.z, v.z, ss);
    ss = fmaf(v.w, v.w, ss);
  }
  const float total = block_sum_256(ss, partial);
  const float inv = 1.0f / sqrtf(total / (float)dim + eps);
  elem_t* dst = out + (size_t)r * dim;
#pragma unroll
  for (int c = 0; c < NORM_CACHED; ++c) {
    const int i = threadIdx.x + c * NORM_THREADS;
    if (i < n4) {
      const int e = i * 4;
      store4(dst + e, (kept[c].x * inv) * load_vec(gain, gain_is_f32, e), (kept[c].y * inv) * load_vec(gain, gain_is_f32, e + 1),
             (kept[c].z * inv) * load_vec(gain, gain_is_f32, e + 2), (kept[c].w * inv) * load_vec(gain, gain_is_f32, e + 3));
    }
  }
  for (int i = threadIdx.x + NORM_CACHED * NORM_THREADS; i < n4; i += NORM_THREADS) {
    const float4 v = src[i];
    const int e = i * 4;
    store4(dst + e, (v.x * inv) * load_vec(gain, gain_is_f32, e), (v.y * inv) * load_vec(gain, gain_is_f32, e + 1),
           (v.z * inv) * load_vec(gain, gain_is_f32, e + 2), (v.w * inv) * load_vec(gain, gain_is_f32, e + 3));
  }
}

// Any width.
__global__ void __launch_bounds__(NORM_THREADS)
rmsnorm_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows, const void* __restrict__ gain,
               int gain_is_f32, elem_t* __restrict__ out, int dim, float eps) {
  __shared__ float partial[NORM_THREADS / AXON_WAVE];
  const int r = blockIdx.x;
  const float* src = x + (size_t)(rows ? rows[r] : r) * dim;
  float ss = 0.0f;
  for (int i = threadIdx.x; i < dim; i += NORM_THREADS) {
    float v = src[i];
    ss = fmaf(v, v, ss);
  }
  const float total = block_sum_256(ss, partial);
  const float ms = total / (float)dim;
  const float inv = 1.0f / sqrtf(ms + eps);
  elem_t* dst = out + (size_t)r * dim;
  for (int i = threadIdx.x; i < dim; i += NORM_THREADS) {
    float g = load_vec(gain, gain_is_f32, i);
    dst[i] = from_float((src[i] * inv) * g);
  }
}

extern "C" int axk_rmsnorm(const float* x, const int32_t* rows, const void* gain, int gain_is_f32, void* out,
                           int n_rows, int dim, float eps, void* stream) {
  AXK_REQUIRE(n_rows >= 0 && dim > 0, "rmsnorm: bad sizes rows=%d dim=%d", n_rows, dim);
  if (n_rows == 0) return 0;
  const bool vec = dim % 4 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)out & 15) == 0;
  if (vec) {
    AXK_INSTANCE(INST_RMSNORM, 1);
    rmsnorm_vec_kernel<<<n_rows, NORM_THREADS, 0, (hipStream_t)stream>>>(x, rows, gain, gain_is_f32, (elem_t*)out, dim,
                                                                        eps);
  } else {
    AXK_INSTANCE(INST_RMSNORM, 0);
    rmsnorm_kernel<<<n_rows, NORM_THREADS, 0, (hipStream_t)stream>>>(x, rows, gain, gain_is_f32, (elem_t*)out, dim, eps);
  }
  AXK_LAUNCH_CHECK("rmsnorm");
  return 0;
}

// ---------------------------------------------------------------------------- rotary tables
// angle = pos * freq_i in float64, (sin, cos) in float64, rounded to float32 once
// (src/model.rs:2612-2621; GPU twin rope_table_b, src/cuda/prefill.cu:60-69).
__global__ void rope_table_kernel(const int32_t* __restrict__ positions, const double* __restrict__ freqs,
                                  float* __restrict__ table, int n_pairs) {
  const int t = blockIdx.x;
  const double pos = (double)positions[t];
  for (int i = threadIdx.x; i < n_pairs; i += blockDim.x) {
    double s, c;
    sincos(pos * freqs[i], &s, &c);
    table[((size_t)t * n_pairs + i) * 2 + 0] = (float)s;
    table[((size_t)t * n_pairs + i) * 2 + 1] = (float)c;
  }
}

extern "C" int axk_rope_table(const int32_t* positions, const double* freqs, float* table, int n_tokens,
                              int n_pairs, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && n_pairs > 0, "rope_table: bad sizes T=%d pairs=%d", n_tokens, n_pairs);
  if (n_tokens == 0) return 0;
  rope_table_kernel<<<n_tokens, 64, 0, (hipStream_t)stream>>>(positions, freqs, table, n_pairs);
  AXK_LAUNCH_CHECK("rope_table");
  return 0;
}

// ---------------------------------------------------------------------------- rotary + cache store
// One wave per (token, head slot), four waves a block: q heads are rotated in place, k heads rotated and stored
// in the request's page for that position, v heads stored as they are (transposed: a page of
// values is [dim][slot], so that the positions of one dim are contiguous).  Pair i of a head
// is (i, i + rotary_dim / 2): out_i = a cos - b sin, out_{i+half} = a sin + b cos, each
// product and sum rounded on its own (src/model.rs:3922-3929; src/cuda/prefill.cu:129-160).
__global__ void rope_kv_write_kernel(elem_t* __restrict__ qkv, const float* __restrict__ table,
                                     const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_rows,
                                     const int32_t* __restrict__ block_table, int table_stride,
                                     elem_t* __restrict__ k_cache, elem_t* __restrict__ v_cache, int n_heads,
                                     int n_kv_heads, int head_dim, int rotary_dim, int page_size, int write_kv) {
  const int t = blockIdx.x;
  const int slot = blockIdx.y * 4 + threadIdx.x / AXON_WAVE;  // 0..nh: q heads; then k heads; then v heads
  const int lane = threadIdx.x % AXON_WAVE;
  if (slot >= n_heads + (write_kv ? 2 * n_kv_heads : 0)) return;
  const int half = rotary_dim / 2;
  const int row_elems = (n_heads + 2 * n_kv_heads) * head_dim;
  elem_t* src = qkv + (size_t)t * row_elems + (size_t)slot * head_dim;
  const float* tab = table + (size_t)t * half * 2;

  elem_t* dst = src;
  if (slot >= n_heads) {
    if (!write_kv) return;
    const int pos = positions[t];
    const int page = block_table[(size_t)seq_rows[t] * table_stride + pos / page_size];
    const int in_page = pos % page_size;
    const bool is_v = slot >= n_heads + n_kv_heads;
    const int kvh = slot - n_heads - (is_v ? n_kv_heads : 0);
    if (is_v) {
      // values are kept position-contiguous: [page][kv head][dim][slot in page]
      elem_t* vdst = v_cache + ((size_t)page * n_kv_heads + kvh) * head_dim * page_size + in_page;
      for (int i = lane; i < head_dim; i += AXON_WAVE) vdst[(size_t)i * page_size] = src[i];
      return;
    }
    dst = k_cache + (((size_t)page * n_kv_heads + kvh) * page_size + in_page) * head_dim;
  }
  for (int i = lane; i < half; i += AXON_WAVE) {
    const float s = tab[2 * i], c = tab[2 * i + 1];
    const float a = to_float(src[i]), b = to_float(src[i + half]);
    const float lo = __fsub_rn(__fmul_rn(a, c), __fmul_rn(b, s));
    const float hi = __fadd_rn(__fmul_rn(a, s), __fmul_rn(b, c));
    dst[i] = from_float(lo);
    dst[i + half] = from_float(hi);
  }
  if (dst != src)
    for (int i = rotary_dim + lane; i < head_dim; i += AXON_WAVE) dst[i] = src[i];
}

extern "C" int axk_rope_kv_write(void* qkv, const float* table, const int32_t* positions, const int32_t* seq_rows,
                                 const int32_t* block_table, int table_stride, void* k_cache, void* v_cache,
                                 int n_tokens, int n_heads, int n_kv_heads, int head_dim, int rotary_dim,
                                 int page_size, int write_kv, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && head_dim > 0 && page_size > 0,
              "rope_kv_write: bad sizes T=%d nh=%d nkv=%d hd=%d page=%d", n_tokens, n_heads, n_kv_heads, head_dim,
              page_size);
  AXK_REQUIRE(rotary_dim >= 0 && rotary_dim <= head_dim && rotary_dim % 2 == 0,
              "rope_kv_write: rotary_dim %d must be even and at most head_dim %d", rotary_dim, head_dim);
  if (n_tokens == 0) return 0;
  dim3 grid(n_tokens, ceil_div(n_heads + (write_kv ? 2 * n_kv_heads : 0), 4));
  rope_kv_write_kernel<<<grid, 4 * AXON_WAVE, 0, (hipStream_t)stream>>>((elem_t*)qkv, table, positions, seq_rows, block_table,
                                                            table_stride, (elem_t*)k_cache, (elem_t*)v_cache,
                                                            n_heads, n_kv_heads, head_dim, rotary_dim, page_size,
                                                            write_kv);
  AXK_LAUNCH_CHECK("rope_kv_write");
  return 0;
}

// ---------------------------------------------------------------------------- SwiGLU
__global__ void swiglu_kernel(const elem_t* __restrict__ gate_up, elem_t* __restrict__ out, int n_ffn) {
  const int t = blockIdx.y;
  const int f = blockIdx.x * blockDim.x + threadIdx.x;
  if (f >= n_ffn) return;
  const elem_t* row = gate_up + (size_t)t * 2 * n_ffn;
  out[(size_t)t * n_ffn + f] = from_float(swiglu1(to_float(row[f]), to_float(row[n_ffn + f])));
}

extern "C" int axk_swiglu(const void* gate_up, void* out, int n_tokens, int n_ffn, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && n_ffn > 0, "swiglu: bad sizes T=%d ffn=%d", n_tokens, n_ffn);
  AXK_REQUIRE(n_tokens <= 65535, "swiglu: %d tokens in one step (at most 65535)", n_tokens);
  if (n_tokens == 0) return 0;
  dim3 grid(ceil_div(n_ffn, 256), n_tokens);
  swiglu_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const elem_t*)gate_up, (elem_t*)out, n_ffn);
  AXK_LAUNCH_CHECK("swiglu");
  return 0;
}

// ---------------------------------------------------------------------------- a norm on a sublayer's output
// x[r, :] += mult * ((y[r, :] * inv_rms(y[r, :])) * gain), and rounded[r, :] = x[r, :] in the compute
// dtype if asked for (what the next sublayer's products read).  The sum of squares as in rmsnorm_kernel.
__global__ void __launch_bounds__(NORM_THREADS)
norm_add_kernel(const float* __restrict__ y, const void* __restrict__ gain, int gain_is_f32, float eps, float mult,
                float* __restrict__ x, elem_t* __restrict__ rounded, int dim) {
  __shared__ float partial[NORM_THREADS / AXON_WAVE];
  const int r = blockIdx.x;
  const float* src = y + (size_t)r * dim;
  float ss = 0.0f;
  for (int i = threadIdx.x; i < dim; i += NORM_THREADS) ss = fmaf(src[i], src[i], ss);
  const float inv = 1.0f / sqrtf(block_sum_256(ss, partial) / (float)dim + eps);
  float* dst = x + (size_t)r * dim;
  for (int i = threadIdx.x; i < dim; i += NORM_THREADS) {
    const float v = dst[i] + mult * ((src[i] * inv) * load_vec(gain, gain_is_f32, i));
    dst[i] = v;
    if (rounded) rounded[(size_t)r * dim + i] = from_float(v);
  }
}

extern "C" int axk_norm_add(const float* y, const void* gain, int gain_is_f32, float eps, float mult, float* x, void* rounded,
                            int n_rows, int dim, void* stream) {
  AXK_REQUIRE(n_rows >= 0 && dim > 0, "norm_add: bad sizes rows=%d dim=%d", n_rows, dim);
  if (n_rows == 0) return 0;
  norm_add_kernel<<<n_rows, NORM_THREADS, 0, (hipStream_t)stream>>>(y, gain, gain_is_f32, eps, mult, x, (elem_t*)rounded, dim);
  AXK_LAUNCH_CHECK("norm_add");
  return 0;
}

// ---------------------------------------------------------------------------- layer norm (a gain, no bias)
// mean = sum x / n, var = sum (x - mean)^2 / n (a second pass over the deviations, not E[x^2] - mean^2),
// out = ((x - mean) * 1 / sqrt(var + eps)) * g.  Both sums as in rmsnorm_kernel: a strided chain per
// thread, a butterfly per wave, the four waves in order.
__global__ void __launch_bounds__(NORM_THREADS)
layernorm_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows, const void* __restrict__ gain,
                 int gain_is_f32, elem_t* __restrict__ out, int dim, float eps) {
  __shared__ float partial[2][NORM_THREADS / AXON_WAVE];
  const int r = blockIdx.x;
  const float* src = x + (size_t)(rows ? rows[r] : r) * dim;
  float sum = 0.0f;
  for (int i = threadIdx.x; i < dim; i += NORM_THREADS) sum += src[i];
  const float mean = block_sum_256(sum, partial[0]) / (float)dim;
  float ss = 0.0f;
  for (int i = threadIdx.x; i < dim; i += NORM_THREADS) {
    const float d = src[i] - mean;
    ss = fmaf(d, d, ss);
  }
  const float inv = 1.0f / sqrtf(block_sum_256(ss, partial[1]) / (float)dim + eps);
  elem_t* dst = out + (size_t)r * dim;
  for (int i = threadIdx.x; i < dim; i += NORM_THREADS)
    dst[i] = from_float(((src[i] - mean) * inv) * load_vec(gain, gain_is_f32, i));
}

extern "C" int axk_layernorm(const float* x, const int32_t* rows, const void* gain, int gain_is_f32, void* out, int n_rows,
                             int dim, float eps, void* stream) {
  AXK_REQUIRE(n_rows >= 0 && dim > 0, "layernorm: bad sizes rows=%d dim=%d", n_rows, dim);
  if (n_rows == 0) return 0;
  layernorm_kernel<<<n_rows, NORM_THREADS, 0, (hipStream_t)stream>>>(x, rows, gain, gain_is_f32, (elem_t*)out, dim, eps);
  AXK_LAUNCH_CHECK("layernorm");
  return 0;
}

// ---------------------------------------------------------------------------- a norm behind the sum
// x[r, :] = norm(alpha x[r, :] + y[r, :]) * gain, the norm an RMS norm (kind 0) or a layer norm (kind 1,
// as layernorm_kernel), and rounded[r, :] = the new x[r, :] in the compute dtype if asked for (what the
// next sublayer's products read).  A thread keeps its first POST_KEPT sums in registers (rows up to
// 4,096 wide are read once); beyond that it adds them again.
#define POST_KEPT 16
__global__ void __launch_bounds__(NORM_THREADS)
sum_norm_kernel(const float* __restrict__ y, float alpha, const void* __restrict__ gain, int gain_is_f32, float eps, int kind,
                float* __restrict__ x, elem_t* __restrict__ rounded, int dim) {
  __shared__ float partial[2][NORM_THREADS / AXON_WAVE];
  const int r = blockIdx.x;
  const float* add = y + (size_t)r * dim;
  float* row = x + (size_t)r * dim;
  float kept[POST_KEPT];
#pragma unroll
  for (int c = 0; c < POST_KEPT; ++c) {
    const int i = threadIdx.x + c * NORM_THREADS;
    kept[c] = i < dim ? alpha * row[i] + add[i] : 0.0f;
  }
  float mean = 0.0f;
  if (kind == 1) {
    float sum = 0.0f;
#pragma unroll
    for (int c = 0; c < POST_KEPT; ++c) sum += kept[c];
    for (int i = threadIdx.x + POST_KEPT * NORM_THREADS; i < dim; i += NORM_THREADS) sum += alpha * row[i] + add[i];
    mean = block_sum_256(sum, partial[0]) / (float)dim;
  }
  float ss = 0.0f;
#pragma unroll
  for (int c = 0; c < POST_KEPT; ++c) {
    const float d = threadIdx.x + c * NORM_THREADS < dim ? kept[c] - mean : 0.0f;
    ss = fmaf(d, d, ss);
  }
  for (int i = threadIdx.x + POST_KEPT * NORM_THREADS; i < dim; i += NORM_THREADS) {
    const float d = (alpha * row[i] + add[i]) - mean;
    ss = fmaf(d, d, ss);
  }
  const float inv = 1.0f / sqrtf(block_sum_256(ss, partial[1]) / (float)dim + eps);
#pragma unroll
  for (int c = 0; c < POST_KEPT; ++c) {
    const int i = threadIdx.x + c * NORM_THREADS;
    if (i < dim) {
      const float v = ((kept[c] - mean) * inv) * load_vec(gain, gain_is_f32, i);
      row[i] = v;
      if (rounded) rounded[(size_t)r * dim + i] = from_float(v);
    }
  }
  for (int i = threadIdx.x + POST_KEPT * NORM_THREADS; i < dim; i += NORM_THREADS) {
    const float v = (((alpha * row[i] + add[i]) - mean) * inv) * load_vec(gain, gain_is_f32, i);
    row[i] = v;
    if (rounded) rounded[(size_t)r * dim + i] = from_float(v);
  }
}

extern "C" int axk_sum_norm(const float* y, float alpha, const void* gain, int gain_is_f32, float eps, int kind, float* x,
                            void* rounded, int n_rows, int dim, void* stream) {
  AXK_REQUIRE(n_rows >= 0 && dim > 0 && (kind == 0 || kind == 1), "sum_norm: bad sizes rows=%d dim=%d kind=%d", n_rows, dim, kind);
  if (n_rows == 0) return 0;
  sum_norm_kernel<<<n_rows, NORM_THREADS, 0, (hipStream_t)stream>>>(y, alpha, gain, gain_is_f32, eps, kind, x, (elem_t*)rounded, dim);
  AXK_LAUNCH_CHECK("sum_norm");
  return 0;
}

// ---------------------------------------------------------------------------- bent logits
// v[r, i] = cap tanh(v[r, i] / cap), in place on float32 rows.
__global__ void softcap_kernel(float* __restrict__ v, long row_stride, int n, float cap) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    float* at = v + (long)blockIdx.y * row_stride + i;
    *at = cap * tanhf(*at / cap);
  }
}

extern "C" int axk_softcap(float* v, long row_stride, int n_rows, int n, float cap, void* stream) {
  AXK_REQUIRE(n_rows >= 0 && n_rows <= 65535 && n > 0 && cap > 0.0f, "softcap: bad sizes rows=%d n=%d cap=%g", n_rows, n, (double)cap);
  if (n_rows == 0) return 0;
  softcap_kernel<<<dim3(ceil_div(n, 256), n_rows), 256, 0, (hipStream_t)stream>>>(v, row_stride, n, cap);
  AXK_LAUNCH_CHECK("softcap");
  return 0;
}

// v[r, i] *= factor, in place on float32 rows.
__global__ void scale_rows_kernel(float* __restrict__ v, long row_stride, int n, float factor) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) v[(long)blockIdx.y * row_stride + i] *= factor;
}

extern "C" int axk_scale_rows(float* v, long row_stride, int n_rows, int n, float factor, void* stream) {
  AXK_REQUIRE(n_rows >= 0 && n_rows <= 65535 && n > 0, "scale_rows: bad sizes rows=%d n=%d", n_rows, n);
  if (n_rows == 0) return 0;
  scale_rows_kernel<<<dim3(ceil_div(n, 256), n_rows), 256, 0, (hipStream_t)stream>>>(v, row_stride, n, factor);
  AXK_LAUNCH_CHECK("scale_rows");
  return 0;
}

// x[i] += factor * y[i] on float32 values (the product is rounded before the sum).
__global__ void add_scaled_kernel(float* __restrict__ x, const float* __restrict__ y, float factor, long n) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] = __fadd_rn(x[i], __fmul_rn(factor, y[i]));
}

extern "C" int axk_add_scaled(float* x, const float* y, float factor, long n, void* stream) {
  if (n <= 0) return 0;
  add_scaled_kernel<<<(unsigned)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(x, y, factor, n);
  AXK_LAUNCH_CHECK("add_scaled");
  return 0;
}

// out[i] = x[i] in the compute dtype.
__global__ void round_rows_kernel(const float* __restrict__ x, elem_t* __restrict__ out, long n) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = from_float(x[i]);
}

extern "C" int axk_round_rows(const float* x, void* out, long n, void* stream) {
  if (n <= 0) return 0;
  round_rows_kernel<<<(unsigned)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(x, (elem_t*)out, n);
  AXK_LAUNCH_CHECK("round_rows");
  return 0;
}

// Two row sets side by side in the compute dtype: out[t, :wa] = a[t, :], out[t, wa:] = b[t, :].
__global__ void concat_round_kernel(const float* __restrict__ a, int wa, const float* __restrict__ b, int wb,
                                    elem_t* __restrict__ out) {
  const long t = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= wa + wb) return;
  out[t * (wa + wb) + i] = from_float(i < wa ? a[t * wa + i] : b[t * wb + i - wa]);
}

extern "C" int axk_concat_round(const float* a, int wa, const float* b, int wb, void* out, int n_rows, void* stream) {
  AXK_REQUIRE(n_rows >= 0 && n_rows <= 65535 * 64 && wa > 0 && wb > 0, "concat_round: bad sizes rows=%d widths %d and %d", n_rows, wa, wb);
  if (n_rows == 0) return 0;
  for (int r0 = 0; r0 < n_rows; r0 += 65535) {
    const int rows = n_rows - r0 < 65535 ? n_rows - r0 : 65535;
    concat_round_kernel<<<dim3((wa + wb + 255) / 256, rows), 256, 0, (hipStream_t)stream>>>(
        a + (long)r0 * wa, wa, b + (long)r0 * wb, wb, (elem_t*)out + (long)r0 * (wa + wb));
  }
  AXK_LAUNCH_CHECK("concat_round");
  return 0;
}

// ---------------------------------------------------------------------------- activations
// In place.  kind 0: the tanh form of GELU, 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)));
// kind 1: the exact GELU, 0.5 z (1 + erf(z / sqrt 2)).
__global__ void activation_kernel(elem_t* __restrict__ v, long n, int kind) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float z = to_float(v[i]);
  if (kind == 1) {
    v[i] = from_float((0.5f * z) * (1.0f + erff(z * 0.7071067811865476f)));
    return;
  }
  const float inner = 0.7978845608028654f * (z + 0.044715f * ((z * z) * z));
  v[i] = from_float((0.5f * z) * (1.0f + tanhf(inner)));
}

extern "C" int axk_activation(void* v, long n, int kind, void* stream) {
  AXK_REQUIRE(kind == 0 || kind == 1, "activation: kind %d is not known (0: gelu, tanh form; 1: gelu, exact)", kind);
  if (n <= 0) return 0;
  activation_kernel<<<(unsigned)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>((elem_t*)v, n, kind);
  AXK_LAUNCH_CHECK("activation");
  return 0;
}

// out[t, f] = g sigmoid(alpha g) (u + 1) with g = min(gu[t, f], limit), u = clamp(gu[t, F + f], -limit, limit).
__global__ void clamped_glu_kernel(const elem_t* __restrict__ gate_up, elem_t* __restrict__ out, int n_ffn, float limit,
                                   float alpha) {
  const int t = blockIdx.y;
  const int f = blockIdx.x * blockDim.x + threadIdx.x;
  if (f >= n_ffn) return;
  const elem_t* row = gate_up + (size_t)t * 2 * n_ffn;
  const float g = fminf(to_float(row[f]), limit);
  const float u = fminf(fmaxf(to_float(row[n_ffn + f]), -limit), limit);
  out[(size_t)t * n_ffn + f] = from_float((g * (1.0f / (1.0f + expf(-(alpha * g))))) * (u + 1.0f));
}

extern "C" int axk_clamped_glu(const void* gate_up, void* out, int n_tokens, int n_ffn, float limit, float alpha, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && n_ffn > 0 && n_tokens <= 65535, "clamped_glu: bad sizes T=%d ffn=%d", n_tokens, n_ffn);
  if (n_tokens == 0) return 0;
  dim3 grid(ceil_div(n_ffn, 256), n_tokens);
  clamped_glu_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const elem_t*)gate_up, (elem_t*)out, n_ffn, limit, alpha);
  AXK_LAUNCH_CHECK("clamped_glu");
  return 0;
}

// ---------------------------------------------------------------------------- fills
template <typename V>
__global__ void fill_kernel(V* dst, V value, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = value;
}

extern "C" int axk_fill_i32(int32_t* dst, int32_t value, int n, void* stream) {
  if (n <= 0) return 0;
  fill_kernel<int32_t><<<ceil_div(n, 256), 256, 0, (hipStream_t)stream>>>(dst, value, n);
  AXK_LAUNCH_CHECK("fill_i32");
  return 0;
}

extern "C" int axk_fill_f32(float* dst, float value, int n, void* stream) {
  if (n <= 0) return 0;
  fill_kernel<float><<<ceil_div(n, 256), 256, 0, (hipStream_t)stream>>>(dst, value, n);
  AXK_LAUNCH_CHECK("fill_f32");
  return 0;
}
