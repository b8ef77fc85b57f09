// Attention over a latent cache: every position keeps one normed latent vector c (rank floats'
// worth, shared by all heads) and one rotated key part (rot floats' worth, shared too).  A head's
// unrotated key is Wuk c and its value Wuv c; neither is ever built.  The query's unrotated part
// is carried into the latent space instead (q_lat = Wuk^T q, a per-head product), so that
//     score(i, j) = (q_lat_i . c_j + q_rot_i . k_rot_j) scale,      o_lat_i = sum_j p_ij c_j,
// and the head's output is Wuv o_lat (another per-head product).  A page of the cache holds its
// positions twice: [page_size][rank + rot] rows (the latent and the rotated key part: what scores
// read), then [rank][page_size], the latents again with the positions of one dim side by side
// (what the matrix cores want as the operand of the weighted sum; the same layout as the values of
// the grouped-query attention's pages).  Scores, weights and sums are 32-bit.
#include "api.h"
#include "common.h"

namespace {

// One block per token.  fused [T, stride] float32 holds the down projections' results:
//   [q_at, q_at + q_rank): the query latent -> RMS norm with q_gain -> cq [T, q_rank] (compute dtype);
//   [kv_at, kv_at + rank): the key/value latent -> RMS norm with kv_gain -> the page;
//   [kv_at + rank, + rot): the shared key part -> its first rot_dims dims rotated -> the page; the pairs are
//   (i, i + rot_dims / 2), or (2i, 2i + 1) with `neighbours`, and cos and sin are multiplied by `magnitude`.
// The sums of squares: a strided chain per thread, a butterfly per wave, the four waves in order.
__global__ void __launch_bounds__(256)
latent_prepare_kernel(const float* __restrict__ fused, long stride, int q_at, int q_rank, int kv_at, int rank, int rot,
                      int rot_dims, int neighbours, float magnitude, const void* __restrict__ q_gain, int q_gain_is_f32,
                      const void* __restrict__ kv_gain, int kv_gain_is_f32, float eps, const float* __restrict__ table, const int32_t* __restrict__ positions,
                      const int32_t* __restrict__ seq_rows, const int32_t* __restrict__ block_table, int table_stride,
                      elem_t* __restrict__ cache, int page_size, elem_t* __restrict__ cq, int write_kv) {
  __shared__ float partial[4];
  const int t = blockIdx.x;
  const float* row = fused + (long)t * stride;
  if (q_rank > 0) {
    float ss = 0.0f;
    for (int i = threadIdx.x; i < q_rank; i += 256) ss = fmaf(row[q_at + i], row[q_at + i], ss);
    const float inv = 1.0f / sqrtf(block_sum_256(ss, partial) / (float)q_rank + eps);
    for (int i = threadIdx.x; i < q_rank; i += 256)
      cq[(long)t * q_rank + i] = from_float((row[q_at + i] * inv) * load_vec(q_gain, q_gain_is_f32, i));
    __syncthreads();
  }
  if (!write_kv) return;
  const int pos = positions[t];
  const int page = block_table[(long)seq_rows[t] * table_stride + pos / page_size];
  elem_t* page_base = cache + (long)page * page_size * (2 * rank + rot);
  elem_t* dst = page_base + (long)(pos % page_size) * (rank + rot);
  elem_t* by_dim = page_base + (long)page_size * (rank + rot) + pos % page_size;      // [rank][page_size]
  float ss = 0.0f;
  for (int i = threadIdx.x; i < rank; i += 256) ss = fmaf(row[kv_at + i], row[kv_at + i], ss);
  const float inv = 1.0f / sqrtf(block_sum_256(ss, partial) / (float)rank + eps);
  for (int i = threadIdx.x; i < rank; i += 256) {
    const elem_t v = from_float((row[kv_at + i] * inv) * load_vec(kv_gain, kv_gain_is_f32, i));
    dst[i] = v;
    by_dim[(long)i * page_size] = v;
  }
  const float* kr = row + kv_at + rank;
  const int half = rot_dims / 2;
  const float* tab = table + (long)t * half * 2;
  for (int i = threadIdx.x; i < half; i += 256) {
    const float s = tab[2 * i] * magnitude, c = tab[2 * i + 1] * magnitude;
    const int ia = neighbours ? 2 * i : i, ib = neighbours ? 2 * i + 1 : i + half;
    const float a = kr[ia], b = kr[ib];
    dst[rank + ia] = from_float(__fsub_rn(__fmul_rn(a, c), __fmul_rn(b, s)));
    dst[rank + ib] = from_float(__fadd_rn(__fmul_rn(b, c), __fmul_rn(a, s)));
  }
  for (int i = rot_dims + threadIdx.x; i < rot; i += 256) dst[rank + i] = from_float(kr[i]);
}

// The rotated part of every head's query: q [T, heads, dim + rot] float32 (rows q_stride apart) -> q_full
// [T, heads, rank + rot] float32, places rank .. rank + rot - 1 (the first `rank` are the per-head
// product's).  Pairs and magnitude as in latent_prepare_kernel.
__global__ void latent_query_rope_kernel(const float* __restrict__ q, long q_stride, int dim, int rot, int rot_dims, int neighbours,
                                         float magnitude, const float* __restrict__ table, float* __restrict__ q_full, int rank,
                                         int heads) {
  const int t = blockIdx.x;
  const int half = rot_dims / 2;
  const float* tab = table + (long)t * half * 2;
  for (int idx = threadIdx.x; idx < heads * rot; idx += blockDim.x) {
    const int h = idx / rot, i = idx % rot;
    const float* src = q + (long)t * q_stride + (long)h * (dim + rot) + dim;
    float v = src[i];
    if (i < rot_dims) {
      const bool first = neighbours ? !(i & 1) : i < half;
      const int pair = neighbours ? i >> 1 : (first ? i : i - half);
      const int other = neighbours ? i ^ 1 : (first ? i + half : i - half);
      const float s = tab[2 * pair] * magnitude, c = tab[2 * pair + 1] * magnitude;
      v = first ? __fsub_rn(__fmul_rn(src[i], c), __fmul_rn(src[other], s)) : __fadd_rn(__fmul_rn(src[i], c), __fmul_rn(src[other], s));
    }
    q_full[((long)t * heads + h) * (rank + rot) + rank + i] = v;
  }
}

// One wave per (token, head), four waves a block.  Positions lo ..= pos in blocks of 64 aligned
// to absolute position, ascending; in a block lane j scores position 64 b + j (walking its key
// row against the query in LDS), the block's maximum and sum are butterflies, and the running
// (m, l, o) are rescaled block by block.  For the values lane d owns the latent dims d, d + 64, ...
// and walks the block's positions, taking each weight from its lane.  `sink` (a number a head, or null):
// the sum of the weights also holds exp(sink) once, which has no key and no value: the running
// (m, l) start at (sink, 1).
#define LA_WAVES 4
__global__ void __launch_bounds__(LA_WAVES * 64)
latent_attention_kernel(const float* __restrict__ q_full, const elem_t* __restrict__ cache,
                        const int32_t* __restrict__ block_table, int table_stride, const int32_t* __restrict__ positions,
                        const int32_t* __restrict__ seq_rows, float* __restrict__ o_lat, int n_tokens, int heads, int rank,
                        int rot, int page_size, int window, float scale, const float* __restrict__ sink) {
  extern __shared__ float smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int width = rank + rot;
  const long page_elems = (long)page_size * (width + rank);
  const long item = (long)blockIdx.x * LA_WAVES + wave;
  const bool active = item < (long)n_tokens * heads;
  const int t = active ? (int)(item / heads) : 0, h = active ? (int)(item % heads) : 0;
  float* qs = smem + (long)wave * width;
  const float* qsrc = q_full + ((long)t * heads + h) * width;
  if (active)
    for (int i = lane; i < width; i += 64) qs[i] = qsrc[i];
  __syncthreads();
  if (!active) return;
  const int pos = positions[t];
  const int lo = window > 0 ? max(0, pos + 1 - window) : 0;
  const int32_t* pages = block_table + (long)seq_rows[t] * table_stride;
  constexpr int MAX_OWN = 16;                      // latent dims a lane owns: rank up to 1024
  float acc[MAX_OWN];
#pragma unroll
  for (int i = 0; i < MAX_OWN; ++i) acc[i] = 0.0f;
  float m = sink ? sink[h] : -INFINITY, l = sink ? 1.0f : 0.0f;
  for (int b = lo / 64; b <= pos / 64; ++b) {
    const int p = b * 64 + lane;
    const bool seen = p >= lo && p <= pos;
    float s = -INFINITY;
    if (seen) {
      const elem_t* key = cache + (long)pages[p / page_size] * page_elems + (long)(p % page_size) * width;
      float dot = 0.0f;
      for (int i = 0; i < width; ++i) dot = fmaf(qs[i], to_float(key[i]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float w = seen ? expf(s - m_new) : 0.0f;
    const float fold = expf(m - m_new);            // 0 at the first block (m = -inf)
    l = fmaf(l, fold, wave_sum(w));
    m = m_new;
#pragma unroll
    for (int i = 0; i < MAX_OWN; ++i) acc[i] *= fold;
    const int j_lo = max(lo, b * 64) - b * 64, j_hi = min(pos, b * 64 + 63) - b * 64;
    for (int j = j_lo; j <= j_hi; ++j) {
      const float wj = __shfl(w, j, 64);
      const int pj = b * 64 + j;
      const elem_t* val = cache + (long)pages[pj / page_size] * page_elems + (long)(pj % page_size) * width;
#pragma unroll
      for (int i = 0; i < MAX_OWN; ++i) {
        const int d = lane + 64 * i;
        if (d < rank) acc[i] = fmaf(wj, to_float(val[d]), acc[i]);
      }
    }
  }
  const float inv = 1.0f / l;
  float* dst = o_lat + ((long)t * heads + h) * rank;
#pragma unroll
  for (int i = 0; i < MAX_OWN; ++i) {
    const int d = lane + 64 * i;
    if (d < rank) dst[d] = acc[i] * inv;
  }
}

#if AXON_BF16
typedef __attribute__((ext_vector_type(8))) __bf16 la_bf16x8;
typedef __attribute__((ext_vector_type(4))) float la_f32x4;
__device__ inline la_bf16x8 la_frag(uint4 v) { return __builtin_bit_cast(la_bf16x8, v); }

// The same attention on the matrix cores.  One wave per (token, sixteen heads), two waves a block,
// each on its own: the sixteen heads of a token see the same positions, so a block of 64 positions is
//   S^T [position, head] = K [position, dims] Q^T           (rank + rot dims in chunks of 32),
//   a maximum, weights and their sum per head (a lane holds 16 positions of its head; the four
//   lanes of a head meet by lane permutation), the running (m, l) and O^T rescaled, then
//   O^T [dim, head] += C^T [dim, position] P^T              (positions in two chunks of 32),
// with K rows and the rows of C^T straight from the page into the first operand (16 or 8 bytes a
// lane) and the rounded weights, as they lie in the accumulators, as the second.  RT: tiles of 16
// latent dims at most; QC: chunks of 32 key dims at most.  Pages hold a multiple of 64 positions.
#define LAM_WAVES 2
template <int RT, int QC, bool SINK>
__global__ void __launch_bounds__(LAM_WAVES * 64)
latent_attention_mfma_kernel(const float* __restrict__ q_full, const bf16_t* __restrict__ cache,
                             const int32_t* __restrict__ block_table, int table_stride, const int32_t* __restrict__ positions,
                             const int32_t* __restrict__ seq_rows, float* __restrict__ o_lat, int n_tokens, int heads, int rank,
                             int rot, int page_size, int window, float scale, const float* __restrict__ sink,
                             float* __restrict__ partial, int n_chunks) {
  // the sixteen heads' queries as bfloat16 in LDS, rows 16 bytes longer than their chunks so that the
  // sixteen rows a product's operand is read from fall into different banks
  constexpr int QROW = QC * 32 + 8;
  __shared__ __align__(16) bf16_t qs_all[LAM_WAVES][16 * QROW];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int groups = heads / 16;
  // without a window the step's last tokens first: they see the most positions, and the waves that start last
  // should be the short ones; over a window most rows are equally long, and the tokens go in their order
  const long n_items = (long)n_tokens * groups, at = (long)blockIdx.x * LAM_WAVES + wave;
  const long item = window > 0 ? at : n_items - 1 - at;
  const bool active = at < n_items;
  const int t = active ? (int)(item / groups) : 0, hg = active ? (int)(item % groups) : 0;
  const int width = rank + rot, qc = width / 32, rt = rank / 16;
  const int j = lane & 15, g = lane >> 4;
  bf16_t* qs = qs_all[wave];
  if (active) {
    const int per_row = width / 8;
    for (int idx = lane; idx < 16 * per_row; idx += 64) {
      const int row = idx / per_row, part = idx % per_row;
      const float* src = q_full + ((long)t * heads + hg * 16 + row) * width + 8 * part;
      const float4 a = *reinterpret_cast<const float4*>(src), b = *reinterpret_cast<const float4*>(src + 4);
      *reinterpret_cast<uint4*>(qs + row * QROW + 8 * part) =
          make_uint4(pack2_bf16(a.x, a.y), pack2_bf16(a.z, a.w), pack2_bf16(b.x, b.y), pack2_bf16(b.z, b.w));
    }
  }
  __syncthreads();
  if (!active) return;
  const bf16_t* qlane = qs + j * QROW + 8 * g;
  const int pos = positions[t];
  const int lo = window > 0 ? max(0, pos + 1 - window) : 0;
  const int32_t* pages = block_table + (long)seq_rows[t] * table_stride;
  const long page_elems = (long)page_size * (width + rank);
  la_f32x4 acc[RT];
#pragma unroll
  for (int i = 0; i < RT; ++i) acc[i] = la_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  // a sink is counted once a row: here when the wave walks all blocks, else by the kernel that folds them
  const bool sunk = SINK && partial == nullptr;        // (an instance of its own: without a sink the running pair starts from constants)
  float m = sunk ? sink[hg * 16 + j] : -INFINITY, l = sunk ? 1.0f : 0.0f;
  // with `partial`: this wave takes one block of 64 positions (blockIdx.y after the token's first) and
  // leaves (o, m, l) unscaled for the kernel that folds a token's blocks in ascending order
  const int b_first = partial ? lo / 64 + (int)blockIdx.y : lo / 64;
  const int b_last = partial ? min(b_first, pos / 64) : pos / 64;
  for (int b = b_first; b <= b_last; ++b) {
    const int p0 = b * 64, in0 = p0 % page_size;
    const bf16_t* page = cache + (long)pages[p0 / page_size] * page_elems;
    const bf16_t* kbase = page + (long)in0 * width + 8 * g;
    const bf16_t* vbase = page + (long)page_size * width + in0 + 4 * g;
    la_f32x4 s[4];
#pragma unroll
    for (int pt = 0; pt < 4; ++pt) {
      s[pt] = la_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
      const bf16_t* krow = kbase + (long)(16 * pt + j) * width;
      constexpr int QB = QC < 10 ? QC : 10;         // chunks of a row asked for before the first product waits for any
#pragma unroll
      for (int k0 = 0; k0 < QC; k0 += QB) {
        uint4 kf[QB];
#pragma unroll
        for (int e = 0; e < QB; ++e)
          if (k0 + e < qc) kf[e] = *reinterpret_cast<const uint4*>(krow + 32 * (k0 + e));
#pragma unroll
        for (int e = 0; e < QB; ++e)
          if (k0 + e < qc) s[pt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(la_frag(kf[e]), la_frag(*reinterpret_cast<const uint4*>(qlane + 32 * (k0 + e))), s[pt], 0, 0, 0);
      }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int pt = 0; pt < 4; ++pt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int p = p0 + 16 * pt + 4 * g + i;
        const float v = (p >= lo && p <= pos) ? s[pt][i] * scale : -INFINITY;
        s[pt][i] = v;
        mx = fmaxf(mx, v);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float fold = expf(m - m_new);
    float sum = 0.0f;
#pragma unroll
    for (int pt = 0; pt < 4; ++pt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float w = expf(s[pt][i] - m_new);        // 0 where the position is not seen
        s[pt][i] = w;
        sum += w;
      }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    l = fmaf(l, fold, sum);
    m = m_new;
    uint4 pf[2];
#pragma unroll
    for (int c = 0; c < 2; ++c)
      pf[c] = make_uint4(pack2_bf16(s[2 * c][0], s[2 * c][1]), pack2_bf16(s[2 * c][2], s[2 * c][3]),
                         pack2_bf16(s[2 * c + 1][0], s[2 * c + 1][1]), pack2_bf16(s[2 * c + 1][2], s[2 * c + 1][3]));
    constexpr int VB = 4;                         // tiles of 16 dims whose rows are asked for together
#pragma unroll
    for (int d0 = 0; d0 < RT; d0 += VB) {
      uint2 v[VB][4];
#pragma unroll
      for (int e = 0; e < VB; ++e) {
        if (d0 + e < rt) {
          const bf16_t* vrow = vbase + (long)(16 * (d0 + e) + j) * page_size;
#pragma unroll
          for (int c = 0; c < 2; ++c) {
            v[e][2 * c] = *reinterpret_cast<const uint2*>(vrow + 32 * c);
            v[e][2 * c + 1] = *reinterpret_cast<const uint2*>(vrow + 32 * c + 16);
          }
        }
      }
#pragma unroll
      for (int e = 0; e < VB; ++e) {
        if (d0 + e < rt) {
          acc[d0 + e] *= fold;
#pragma unroll
          for (int c = 0; c < 2; ++c)
            acc[d0 + e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                la_frag(make_uint4(v[e][2 * c].x, v[e][2 * c].y, v[e][2 * c + 1].x, v[e][2 * c + 1].y)), la_frag(pf[c]), acc[d0 + e],
                0, 0, 0);
        }
      }
    }
  }
  if (partial) {
    float* dst = partial + (((long)t * heads + hg * 16 + j) * n_chunks + blockIdx.y) * (rank + 2);
#pragma unroll
    for (int dt = 0; dt < RT; ++dt)
      if (dt < rt) *reinterpret_cast<float2*>(dst + 16 * dt + 4 * g) = make_float2(acc[dt][0], acc[dt][1]),
                   *reinterpret_cast<float2*>(dst + 16 * dt + 4 * g + 2) = make_float2(acc[dt][2], acc[dt][3]);
    if (g == 0) { dst[rank] = m; dst[rank + 1] = l; }
    return;
  }
  const float inv = 1.0f / l;
  float* dst = o_lat + ((long)t * heads + hg * 16 + j) * rank + 4 * g;
#pragma unroll
  for (int dt = 0; dt < RT; ++dt)
    if (dt < rt) *reinterpret_cast<float4*>(dst + 16 * dt) = make_float4(acc[dt][0] * inv, acc[dt][1] * inv, acc[dt][2] * inv, acc[dt][3] * inv);
}

// The same for steps of many tokens: four waves a block take four neighbouring tokens (and the same sixteen
// heads).  Where these belong to one request (a prompt's portion) they read the same pages, and a block of
// 64 positions is staged in LDS once for the four: its K rows [64][rank + rot] for the scores, then, in the
// same buffer, its C^T rows [rank][64] for the weighted sums (rows 16 bytes longer than their content, as the
// queries').  Each wave keeps its own mask, running pair and accumulators, and runs the chain of products
// of the kernel above: the same bits.  Tokens of several requests in one block (decoding rows side by
// side): every wave reads its own pages from memory, as above.
#define LAS_WAVES 4
#define LATENT_TOKENS_KERNEL_FROM 256           // (token, sixteen heads) items of a step from which four tokens share a block
template <int RT, int QC, bool SHARED>
__device__ __forceinline__ void latent_walk(const bf16_t* __restrict__ cache, const int32_t* __restrict__ pages, long page_elems,
                                            int page_size, int width, int rank, int qc, int rt, int b_from, int b_to, bool active,
                                            int lo, int pos, float scale, const bf16_t* qlane, bf16_t* stage, int j, int g,
                                            float& m, float& l, la_f32x4 (&acc)[RT]) {
  const int KROW = width + 8;
  constexpr int VROW = 64 + 8;
  for (int b = b_from; b <= b_to; ++b) {
    const int p0 = b * 64, in0 = p0 % page_size;
    const bf16_t* page = cache + (long)pages[p0 / page_size] * page_elems;
    const bool mine = active && b >= lo / 64 && b <= pos / 64;
    const bf16_t* kbase;
    long krow_stride;
    if constexpr (SHARED) {
      __syncthreads();                               // the buffer's last readers are done
      const uint4* src = reinterpret_cast<const uint4*>(page + (long)in0 * width);
      const int per_row = width / 8, units = 64 * per_row;
      {
        // every load of the block's K rows in flight at once (the registers of the scores are free here)
        uint4 held[QC];
#pragma unroll
        for (int e = 0; e < QC; ++e)
          held[e] = src[min((int)threadIdx.x + e * LAS_WAVES * 64, units - 1)];
#pragma unroll
        for (int e = 0; e < QC; ++e) {
          const int u = threadIdx.x + e * LAS_WAVES * 64;
          if (u < units) *reinterpret_cast<uint4*>(stage + (u / per_row) * KROW + 8 * (u % per_row)) = held[e];
        }
      }
      __syncthreads();
      kbase = stage + 8 * g;
      krow_stride = KROW;
    } else {
      kbase = page + (long)in0 * width + 8 * g;
      krow_stride = width;
    }
    la_f32x4 s[4];
    uint4 pf[2];
    float fold = 1.0f;
    if (mine) {
#pragma unroll
      for (int pt = 0; pt < 4; ++pt) {
        s[pt] = la_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        const bf16_t* krow = kbase + (long)(16 * pt + j) * krow_stride;
        constexpr int QB = SHARED ? (QC < 4 ? QC : 4) : (QC < 10 ? QC : 10);
#pragma unroll
        for (int k0 = 0; k0 < QC; k0 += QB) {
          uint4 kf[QB];
#pragma unroll
          for (int e = 0; e < QB; ++e)
            if (k0 + e < qc) kf[e] = *reinterpret_cast<const uint4*>(krow + 32 * (k0 + e));
#pragma unroll
          for (int e = 0; e < QB; ++e)
            if (k0 + e < qc) s[pt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(la_frag(kf[e]), la_frag(*reinterpret_cast<const uint4*>(qlane + 32 * (k0 + e))), s[pt], 0, 0, 0);
        }
      }
      float mx = -INFINITY;
#pragma unroll
      for (int pt = 0; pt < 4; ++pt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int p = p0 + 16 * pt + 4 * g + i;
          const float v = (p >= lo && p <= pos) ? s[pt][i] * scale : -INFINITY;
          s[pt][i] = v;
          mx = fmaxf(mx, v);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m, mx);
      fold = expf(m - m_new);
      float sum = 0.0f;
#pragma unroll
      for (int pt = 0; pt < 4; ++pt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float w = expf(s[pt][i] - m_new);        // 0 where the position is not seen
          s[pt][i] = w;
          sum += w;
        }
      sum += __shfl_xor(sum, 16, 64);
      sum += __shfl_xor(sum, 32, 64);
      l = fmaf(l, fold, sum);
      m = m_new;
#pragma unroll
      for (int c = 0; c < 2; ++c)
        pf[c] = make_uint4(pack2_bf16(s[2 * c][0], s[2 * c][1]), pack2_bf16(s[2 * c][2], s[2 * c][3]),
                           pack2_bf16(s[2 * c + 1][0], s[2 * c + 1][1]), pack2_bf16(s[2 * c + 1][2], s[2 * c + 1][3]));
    }
    const bf16_t* vbase;
    long vrow_stride;
    if constexpr (SHARED) {
      __syncthreads();                               // the K rows' readers are done
      const bf16_t* src = page + (long)page_size * width + in0;
      const int units = rank * 8;
      {
        constexpr int VU = (RT + 1) / 2;             // rank x 8 units of 16 bytes over 256 threads
        uint4 held[VU];
#pragma unroll
        for (int e = 0; e < VU; ++e) {
          const int u = min((int)threadIdx.x + e * LAS_WAVES * 64, units - 1);
          held[e] = *reinterpret_cast<const uint4*>(src + (long)(u / 8) * page_size + 8 * (u % 8));
        }
#pragma unroll
        for (int e = 0; e < VU; ++e) {
          const int u = threadIdx.x + e * LAS_WAVES * 64;
          if (u < units) *reinterpret_cast<uint4*>(stage + (u / 8) * VROW + 8 * (u % 8)) = held[e];
        }
      }
      __syncthreads();
      vbase = stage + 4 * g;
      vrow_stride = VROW;
    } else {
      vbase = page + (long)page_size * width + in0 + 4 * g;
      vrow_stride = page_size;
    }
    if (mine) {
      constexpr int VB = SHARED ? 2 : 4;             // tiles of 16 dims whose rows are asked for together
#pragma unroll
      for (int d0 = 0; d0 < RT; d0 += VB) {
        uint2 v[VB][4];
#pragma unroll
        for (int e = 0; e < VB; ++e) {
          if (d0 + e < rt) {
            const bf16_t* vrow = vbase + (long)(16 * (d0 + e) + j) * vrow_stride;
#pragma unroll
            for (int c = 0; c < 2; ++c) {
              v[e][2 * c] = *reinterpret_cast<const uint2*>(vrow + 32 * c);
              v[e][2 * c + 1] = *reinterpret_cast<const uint2*>(vrow + 32 * c + 16);
            }
          }
        }
#pragma unroll
        for (int e = 0; e < VB; ++e) {
          if (d0 + e < rt) {
            acc[d0 + e] *= fold;
#pragma unroll
            for (int c = 0; c < 2; ++c)
              acc[d0 + e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                  la_frag(make_uint4(v[e][2 * c].x, v[e][2 * c].y, v[e][2 * c + 1].x, v[e][2 * c + 1].y)), la_frag(pf[c]), acc[d0 + e],
                  0, 0, 0);
          }
        }
      }
    }
  }
}

template <int RT, int QC, bool SINK>
__global__ void __launch_bounds__(LAS_WAVES * 64)
latent_attention_mfma_tokens_kernel(const float* __restrict__ q_full, const bf16_t* __restrict__ cache,
                                    const int32_t* __restrict__ block_table, int table_stride, const int32_t* __restrict__ positions,
                                    const int32_t* __restrict__ seq_rows, float* __restrict__ o_lat, int n_tokens, int heads, int rank,
                                    int rot, int page_size, int window, float scale, const float* __restrict__ sink) {
  extern __shared__ __align__(16) bf16_t las_lds[];
  bf16_t* stage = las_lds;                                                        // max(64 x (width + 8), rank x 72) elements
  const int QROW = rank + rot + 8;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  bf16_t* qs = las_lds + max(64 * QROW, rank * 72) + wave * 16 * QROW;
  const int groups = heads / 16;
  const int n_tiles = (n_tokens + LAS_WAVES - 1) / LAS_WAVES;
  // without a window the step's last tokens first (see the kernel above)
  const int at = (int)blockIdx.x / groups, hg = (int)blockIdx.x % groups;
  const int tile = window > 0 ? at : n_tiles - 1 - at;
  const int t = tile * LAS_WAVES + wave;
  const bool active = t < n_tokens;
  const int width = rank + rot, qc = width / 32, rt = rank / 16;
  const int j = lane & 15, g = lane >> 4;
  if (active) {
    const int per_row = width / 8;
    for (int idx = lane; idx < 16 * per_row; idx += 64) {
      const int row = idx / per_row, part = idx % per_row;
      const float* src = q_full + ((long)t * heads + hg * 16 + row) * width + 8 * part;
      const float4 a = *reinterpret_cast<const float4*>(src), b = *reinterpret_cast<const float4*>(src + 4);
      *reinterpret_cast<uint4*>(qs + row * QROW + 8 * part) =
          make_uint4(pack2_bf16(a.x, a.y), pack2_bf16(a.z, a.w), pack2_bf16(b.x, b.y), pack2_bf16(b.z, b.w));
    }
  }
  // the block's tokens: one request (its pages staged once for all) or several (every wave on its own)
  const int t_first = tile * LAS_WAVES, t_last = min(t_first + LAS_WAVES, n_tokens) - 1;
  bool same = true;
  int b_from = 1 << 30, b_to = -1;
  for (int u = t_first; u <= t_last; ++u) {
    same = same && seq_rows[u] == seq_rows[t_first];
    const int p = positions[u];
    b_from = min(b_from, (window > 0 ? max(0, p + 1 - window) : 0) / 64);
    b_to = max(b_to, p / 64);
  }
  const bf16_t* qlane = qs + j * QROW + 8 * g;
  const int pos = active ? positions[t] : 0;
  const int lo = window > 0 ? max(0, pos + 1 - window) : 0;
  const int32_t* pages = block_table + (long)seq_rows[active ? t : t_first] * table_stride;
  const long page_elems = (long)page_size * (width + rank);
  la_f32x4 acc[RT];
#pragma unroll
  for (int i = 0; i < RT; ++i) acc[i] = la_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  float m = (SINK && active) ? sink[hg * 16 + j] : -INFINITY, l = SINK ? 1.0f : 0.0f;
  __syncthreads();
  if (same)
    latent_walk<RT, QC, true>(cache, pages, page_elems, page_size, width, rank, qc, rt, b_from, b_to, active, lo, pos, scale, qlane, stage,
                              j, g, m, l, acc);
  else if (active)
    latent_walk<RT, QC, false>(cache, pages, page_elems, page_size, width, rank, qc, rt, lo / 64, pos / 64, true, lo, pos, scale, qlane,
                               stage, j, g, m, l, acc);
  if (!active) return;
  const float inv = 1.0f / l;
  float* dst = o_lat + ((long)t * heads + hg * 16 + j) * rank + 4 * g;
#pragma unroll
  for (int dt = 0; dt < RT; ++dt)
    if (dt < rt) *reinterpret_cast<float4*>(dst + 16 * dt) = make_float4(acc[dt][0] * inv, acc[dt][1] * inv, acc[dt][2] * inv, acc[dt][3] * inv);
}

// o_lat[row, :] = sum_c exp(m_c - M) o_c / sum_c exp(m_c - M) l_c over a row's blocks in ascending order
// (M the largest m_c; a block that saw nothing has l = 0 and weighs nothing).  One block per (token,
// head): the blocks' (m, l) once into LDS, all loads in flight together, their weights from there, then
// a thread a dim whose chain over the blocks has eight loads in flight.  With a sink, M is at least the
// head's sink and the sum of the weights holds exp(sink - M) as well.
__global__ void __launch_bounds__(512)
latent_attention_fold_kernel(const float* __restrict__ partial, float* __restrict__ o_lat, int rank, int n_chunks,
                             const float* __restrict__ sink, int heads) {
  extern __shared__ float fold_lds[];
  float* weight = fold_lds;
  float* ms = fold_lds + n_chunks;
  float* ls = ms + n_chunks;
  const float* src = partial + (long)blockIdx.x * n_chunks * (rank + 2);
  for (int c = threadIdx.x; c < n_chunks; c += blockDim.x) {
    ms[c] = src[(long)c * (rank + 2) + rank];
    ls[c] = src[(long)c * (rank + 2) + rank + 1];
  }
  __syncthreads();
  float M = sink ? sink[blockIdx.x % heads] : -INFINITY;
  for (int c = 0; c < n_chunks; ++c)
    if (ls[c] > 0.0f) M = fmaxf(M, ms[c]);
  for (int c = threadIdx.x; c < n_chunks; c += blockDim.x) weight[c] = ls[c] > 0.0f ? expf(ms[c] - M) : 0.0f;
  __syncthreads();
  float L = sink ? expf(sink[blockIdx.x % heads] - M) : 0.0f;
  for (int c = 0; c < n_chunks; ++c) L = fmaf(weight[c], ls[c], L);
  const float inv = 1.0f / L;
  for (int d = threadIdx.x; d < rank; d += blockDim.x) {
    float o = 0.0f;
#pragma unroll 8
    for (int c = 0; c < n_chunks; ++c) o = fmaf(weight[c], src[(long)c * (rank + 2) + d], o);
    o_lat[(long)blockIdx.x * rank + d] = o * inv;
  }
}

// Steps of many tokens (no blocks side by side): four tokens a block, their pages staged in LDS once.
static long latent_tokens_lds(int rank, int rot) {
  const long qrow = rank + rot + 8, stage = 64 * qrow > (long)rank * 72 ? 64 * qrow : (long)rank * 72;
  return (stage + LAS_WAVES * 16 * qrow) * (long)sizeof(bf16_t);
}
#define LATENT_LDS_MOST (160 * 1024)

template <int RT, int QC>
static int launch_latent_mfma_tokens(const float* q_full, const void* cache, const int32_t* block_table, int table_stride,
                                     const int32_t* positions, const int32_t* seq_rows, float* o_lat, int n_tokens, int heads, int rank,
                                     int rot, int page_size, int window, float scale, const float* sink, hipStream_t stream) {
  const int lds = (int)latent_tokens_lds(rank, rot);
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&latent_attention_mfma_tokens_kernel<RT, QC, true>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, LATENT_LDS_MOST);
    if (e == hipSuccess)
      e = hipFuncSetAttribute(reinterpret_cast<const void*>(&latent_attention_mfma_tokens_kernel<RT, QC, false>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, LATENT_LDS_MOST);
    if (e != hipSuccess) {
      axk_set_error("latent_attention: cannot reserve %d bytes of LDS: %s", LATENT_LDS_MOST, hipGetErrorString(e));
      return -2;
    }
    configured = true;
  }
  const unsigned grid = (unsigned)(((n_tokens + LAS_WAVES - 1) / LAS_WAVES) * (heads / 16));
  if (sink)
    latent_attention_mfma_tokens_kernel<RT, QC, true><<<grid, LAS_WAVES * 64, lds, stream>>>(
        q_full, (const bf16_t*)cache, block_table, table_stride, positions, seq_rows, o_lat, n_tokens, heads, rank, rot, page_size, window,
        scale, sink);
  else
    latent_attention_mfma_tokens_kernel<RT, QC, false><<<grid, LAS_WAVES * 64, lds, stream>>>(
        q_full, (const bf16_t*)cache, block_table, table_stride, positions, seq_rows, o_lat, n_tokens, heads, rank, rot, page_size, window,
        scale, sink);
  return 0;
}

template <int RT, int QC>
static void launch_latent_mfma(const float* q_full, const void* cache, const int32_t* block_table, int table_stride,
                               const int32_t* positions, const int32_t* seq_rows, float* o_lat, int n_tokens, int heads, int rank,
                               int rot, int page_size, int window, float scale, const float* sink, float* partial, int n_chunks,
                               hipStream_t stream) {
  const long items = (long)n_tokens * (heads / 16);
  dim3 grid((unsigned)((items + LAM_WAVES - 1) / LAM_WAVES), partial ? n_chunks : 1);
  if (sink)
    latent_attention_mfma_kernel<RT, QC, true><<<grid, LAM_WAVES * 64, 0, stream>>>(
        q_full, (const bf16_t*)cache, block_table, table_stride, positions, seq_rows, o_lat, n_tokens, heads, rank, rot, page_size,
        window, scale, sink, partial, n_chunks);
  else
    latent_attention_mfma_kernel<RT, QC, false><<<grid, LAM_WAVES * 64, 0, stream>>>(
        q_full, (const bf16_t*)cache, block_table, table_stride, positions, seq_rows, o_lat, n_tokens, heads, rank, rot, page_size,
        window, scale, sink, partial, n_chunks);
  if (partial)
    latent_attention_fold_kernel<<<n_tokens * heads, min(512, (rank + 63) / 64 * 64), 3 * n_chunks * sizeof(float), stream>>>(
        partial, o_lat, rank, n_chunks, sink, heads);
}
#endif

}  // namespace

// 1 where axk_latent_attention runs on the matrix cores (the bfloat16 build, heads in sixteens,
// a latent in sixteens up to 512, key rows in chunks of 32 up to 640, pages of a multiple of 64).
extern "C" int axk_latent_attention_uses_mfma(int heads, int rank, int rot, int page_size) {
#if AXON_BF16
  return heads % 16 == 0 && rank % 16 == 0 && (rank + rot) % 32 == 0 && page_size % 64 == 0 && rank <= 512 && rank + rot <= 640;
#else
  return 0;
#endif
}

extern "C" int axk_latent_prepare(const float* fused, long stride, int q_at, int q_rank, int kv_at, int rank, int rot,
                                  int rot_dims, int neighbours, float magnitude, const void* q_gain, int q_gain_is_f32, const void* kv_gain,
                                  int kv_gain_is_f32, float eps, const float* table, const int32_t* positions,
                                  const int32_t* seq_rows, const int32_t* block_table, int table_stride, void* cache,
                                  int page_size, void* cq, int n_tokens, int write_kv, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && q_rank >= 0 && rank > 0 && rot >= 0 && page_size > 0, "latent_prepare: bad sizes T=%d q_rank=%d "
              "rank=%d rot=%d page=%d", n_tokens, q_rank, rank, rot, page_size);
  AXK_REQUIRE(rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0, "latent_prepare: %d rotated dims of %d", rot_dims, rot);
  AXK_REQUIRE(q_at >= 0 && kv_at >= 0 && q_at + q_rank <= stride && kv_at + rank + rot <= stride,
              "latent_prepare: the parts do not fit rows of %ld", stride);
  if (n_tokens == 0) return 0;
  latent_prepare_kernel<<<n_tokens, 256, 0, (hipStream_t)stream>>>(fused, stride, q_at, q_rank, kv_at, rank, rot, rot_dims,
      neighbours, magnitude, q_gain, q_gain_is_f32, kv_gain, kv_gain_is_f32, eps, table, positions, seq_rows, block_table, table_stride,
      (elem_t*)cache, page_size, (elem_t*)cq, write_kv);
  AXK_LAUNCH_CHECK("latent_prepare");
  return 0;
}

extern "C" int axk_latent_query_rope(const float* q, long q_stride, int dim, int rot, int rot_dims, int neighbours, float magnitude,
                                     const float* table, float* q_full, int rank, int heads, int n_tokens, void* stream) {
  AXK_REQUIRE(q_stride >= (long)heads * (dim + rot), "latent_query_rope: rows %ld apart hold no %d heads of %d", q_stride, heads,
              dim + rot);
  AXK_REQUIRE(n_tokens >= 0 && dim >= 0 && rot >= 0 && rank > 0 && heads > 0 && rot_dims % 2 == 0 && rot_dims <= rot,
              "latent_query_rope: bad sizes T=%d dim=%d rot=%d (%d rotated) rank=%d heads=%d", n_tokens, dim, rot, rot_dims,
              rank, heads);
  if (n_tokens == 0 || rot == 0) return 0;
  latent_query_rope_kernel<<<n_tokens, 256, 0, (hipStream_t)stream>>>(q, q_stride, dim, rot, rot_dims, neighbours, magnitude, table, q_full,
                                                                      rank, heads);
  AXK_LAUNCH_CHECK("latent_query_rope");
  return 0;
}

// Few tokens (a decoding step): a wave per block of 64 positions, so that the blocks of a token run side
// by side; the floats of the workspace this takes (0: the tokens' waves walk their blocks themselves).
// A window of w positions touches at most (w + 62) / 64 + 1 blocks; without a window the caller says how
// many positions the longest row of the step sees (`span`; 0: not known, no blocks side by side).
static int latent_blocks_side_by_side(int window, int span) {
  if (window > 0 && (span <= 0 || span > window)) return (window + 62) / 64 + 1;
  return span > 0 ? (span + 63) / 64 : 0;
}

extern "C" long axk_latent_attention_workspace(int n_tokens, int heads, int rank, int rot, int page_size, int window, int span) {
  if (!axk_latent_attention_uses_mfma(heads, rank, rot, page_size)) return 0;
  const int blocks = latent_blocks_side_by_side(window, span);
  if (blocks < 2 || (long)n_tokens * (heads / 16) >= 512) return 0;
  return (long)n_tokens * heads * blocks * (rank + 2);
}

extern "C" int axk_latent_attention(const float* q_full, const void* cache, const int32_t* block_table, int table_stride,
                                    const int32_t* positions, const int32_t* seq_rows, float* o_lat, int n_tokens, int heads,
                                    int rank, int rot, int page_size, int window, int span, float scale, const float* sink,
                                    float* partial, long partial_floats, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && heads > 0 && rank > 0 && rot >= 0 && page_size > 0 && window >= 0,
              "latent_attention: bad sizes T=%d heads=%d rank=%d rot=%d page=%d window=%d", n_tokens, heads, rank, rot,
              page_size, window);
  AXK_REQUIRE(rank <= 1024, "latent_attention: a latent of %d dims (at most 1024)", rank);
  AXK_REQUIRE((long)(rank + rot) * LA_WAVES * 4 <= 64 * 1024, "latent_attention: keys of %d dims do not fit LDS", rank + rot);
  if (n_tokens == 0) return 0;
#if AXON_BF16
  if (axk_latent_attention_uses_mfma(heads, rank, rot, page_size) && ((uintptr_t)q_full & 15) == 0 && ((uintptr_t)cache & 15) == 0 &&
      ((uintptr_t)o_lat & 15) == 0) {
    hipStream_t s = (hipStream_t)stream;
    const long need = axk_latent_attention_workspace(n_tokens, heads, rank, rot, page_size, window, span);
    AXK_REQUIRE(partial == nullptr || partial_floats >= need, "latent_attention: a workspace of %ld floats, %ld needed",
                partial_floats, need);
    if (need == 0) partial = nullptr;
    const int n_chunks = latent_blocks_side_by_side(window, span);
    if (partial == nullptr && (long)n_tokens * (heads / 16) >= LATENT_TOKENS_KERNEL_FROM && latent_tokens_lds(rank, rot) <= LATENT_LDS_MOST) {
      int rc;
      if (rank <= 64 && rank + rot <= 128)
        rc = launch_latent_mfma_tokens<4, 4>(q_full, cache, block_table, table_stride, positions, seq_rows, o_lat, n_tokens, heads, rank,
                                             rot, page_size, window, scale, sink, s);
      else if (rank <= 128 && rank + rot <= 256)
        rc = launch_latent_mfma_tokens<8, 8>(q_full, cache, block_table, table_stride, positions, seq_rows, o_lat, n_tokens, heads, rank,
                                             rot, page_size, window, scale, sink, s);
      else
        rc = launch_latent_mfma_tokens<32, 20>(q_full, cache, block_table, table_stride, positions, seq_rows, o_lat, n_tokens, heads,
                                               rank, rot, page_size, window, scale, sink, s);
      if (rc) return rc;
      AXK_LAUNCH_CHECK("latent_attention");
      return 0;
    }
    if (rank <= 64 && rank + rot <= 128)
      launch_latent_mfma<4, 4>(q_full, cache, block_table, table_stride, positions, seq_rows, o_lat, n_tokens, heads, rank, rot,
                               page_size, window, scale, sink, partial, n_chunks, s);
    else if (rank <= 128 && rank + rot <= 256)
      launch_latent_mfma<8, 8>(q_full, cache, block_table, table_stride, positions, seq_rows, o_lat, n_tokens, heads, rank, rot,
                               page_size, window, scale, sink, partial, n_chunks, s);
    else
      launch_latent_mfma<32, 20>(q_full, cache, block_table, table_stride, positions, seq_rows, o_lat, n_tokens, heads, rank, rot,
                                 page_size, window, scale, sink, partial, n_chunks, s);
    AXK_LAUNCH_CHECK("latent_attention");
    return 0;
  }
#endif
  const long items = (long)n_tokens * heads;
  const size_t lds = (size_t)(rank + rot) * LA_WAVES * sizeof(float);
  latent_attention_kernel<<<(unsigned)((items + LA_WAVES - 1) / LA_WAVES), LA_WAVES * 64, lds, (hipStream_t)stream>>>(
      q_full, (const elem_t*)cache, block_table, table_stride, positions, seq_rows, o_lat, n_tokens, heads, rank, rot,
      page_size, window, scale, sink);
  AXK_LAUNCH_CHECK("latent_attention");
  return 0;
}
