// Grouped-query attention with the variations a configuration may ask for, each a parameter:
//   * one or two score maps a head (two: differential attention, o = rms(a_1 - lambda a_2) c over one
//     set of values), keys of `dim` and values of `vdim` elements, `heads` query heads over `kv_heads`;
//   * a per-head RMS norm of queries and keys with a gain, rotation of the leading dims in either
//     pairing (places (2i, 2i + 1) or (i, i + n / 2)) with cos and sin scaled by a factor;
//   * what a position sees: every earlier position, the last `size` positions (a sliding window), or
//     the earlier positions of its own chunk of `size` (chunks counted from position 0);
//   * scores bent by cap tanh(s / cap);
//   * a sink in the softmax: a key of a given score that has no value (its weight only enters the sum);
//   * a query temperature by position, q (1 + coef ln(floor((p + 1) / every) + 1));
//   * a gate sigmoid(g) on the concatenated heads, a number an element or a number a head.
//
// A page of the cache holds, for its positions, the key rows [page_size][kv_heads maps dim] and behind
// them the values with the positions of one dim side by side, [kv_heads vdim][page_size] (the operand
// layout of the matrix cores' weighted sum).  Scores, weights, sums and norms are 32-bit in both builds.
#include <math.h>

#include "api.h"
#include "common.h"

namespace {

enum { MASK_CAUSAL = 0, MASK_WINDOW = 1, MASK_CHUNK = 2 };

__device__ inline int first_seen(int pos, int mask_kind, int mask_size) {
  if (mask_kind == MASK_WINDOW) return max(0, pos + 1 - mask_size);
  if (mask_kind == MASK_CHUNK) return pos / mask_size * mask_size;
  return 0;
}

// One block per token (or several side by side, each with its share of the units), a wave a unit (one map of one head) at a time.  proj [T, stride] float32 holds
// the projections' results: n_q units of `dim` from q_at, n_k units from k_at, and v_width values from
// v_at (v_at may equal k_at: the values are the keys as projected).  Units are RMS-normed with a gain
// shared by all units (if given), their first rot dims rotated by the step's table [T, rot / 2, 2]
// (sin, cos), and stored: queries into q_out [T, n_q dim], keys and values into the token's page.
__global__ void __launch_bounds__(256)
heads_prepare_kernel(const float* __restrict__ proj, long stride, int q_at, int n_q, int k_at, int n_k, int v_at, int v_width,
                     int dim, const void* __restrict__ q_gain, int q_gain_is_f32, const void* __restrict__ k_gain,
                     int k_gain_is_f32, float eps, int rot, int neighbours, float magnitude, const float* __restrict__ table,
                     const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_rows,
                     const int32_t* __restrict__ block_table, int table_stride, elem_t* __restrict__ cache, int page_size,
                     elem_t* __restrict__ q_out, int write_kv, float q_temp_coef, int q_temp_every) {
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  // a query's temperature by its position: 1 + coef ln(floor((p + 1) / every) + 1), or 1
  const float q_temp = q_temp_every > 0 ? 1.0f + q_temp_coef * logf((float)((positions[t] + 1) / q_temp_every + 1)) : 1.0f;
  const float* row = proj + (long)t * stride;
  const int half = rot / 2;
  const float* tab = table + (long)t * half * 2;
  const int kw = n_k * dim;
  elem_t* page_base = nullptr;
  int in_page = 0;
  if (write_kv) {
    const int pos = positions[t];
    const int page = block_table[(long)seq_rows[t] * table_stride + pos / page_size];
    page_base = cache + (long)page * page_size * (kw + v_width);
    in_page = pos % page_size;
  }
  const int n_units = n_q + (write_kv ? n_k : 0);
  for (int u = blockIdx.y * 4 + wave; u < n_units; u += 4 * gridDim.y) {
    const bool is_q = u < n_q;
    const float* src = row + (is_q ? q_at + u * dim : k_at + (u - n_q) * dim);
    elem_t* dst = is_q ? q_out + ((long)t * n_q + u) * dim : page_base + (long)in_page * kw + (long)(u - n_q) * dim;
    const void* gain = is_q ? q_gain : k_gain;
    const int gain_is_f32 = is_q ? q_gain_is_f32 : k_gain_is_f32;
    const float temp = is_q ? q_temp : 1.0f;
    float inv = 1.0f;
    if (gain != nullptr) {
      float ss = 0.0f;
      for (int i = lane; i < dim; i += 64) ss = fmaf(src[i], src[i], ss);
      inv = 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps);
    }
    for (int i = lane; i < half; i += 64) {
      const int ia = neighbours ? 2 * i : i, ib = neighbours ? 2 * i + 1 : i + half;
      float a = src[ia], b = src[ib];
      if (gain != nullptr) {
        a = (a * inv) * load_vec(gain, gain_is_f32, ia);
        b = (b * inv) * load_vec(gain, gain_is_f32, ib);
      }
      const float s = tab[2 * i] * magnitude, c = tab[2 * i + 1] * magnitude;
      dst[ia] = from_float(__fsub_rn(__fmul_rn(a, c), __fmul_rn(b, s)) * temp);
      dst[ib] = from_float(__fadd_rn(__fmul_rn(b, c), __fmul_rn(a, s)) * temp);
    }
    for (int i = rot + lane; i < dim; i += 64) {
      float a = src[i];
      if (gain != nullptr) a = (a * inv) * load_vec(gain, gain_is_f32, i);
      dst[i] = from_float(a * temp);
    }
  }
  if (!write_kv) return;
  elem_t* by_dim = page_base + (long)page_size * kw + in_page;
  for (int i = blockIdx.y * 256 + threadIdx.x; i < v_width; i += 256 * gridDim.y) by_dim[(long)i * page_size] = from_float(row[v_at + i]);
}

// One wave per (token, head), four waves a block; any sizes, both builds.  For each map: positions
// first ..= pos in blocks of 64 aligned to absolute position, ascending; lane j scores position
// 64 b + j against the query in LDS, the block's maximum and sum are butterflies, and the running
// (m, l, o) are rescaled block by block; lane d owns value dims d, d + 64, ...  Then the maps are
// combined, normed and gated, and the head's vdim outputs stored.
#define MA_WAVES 4
#define MA_OWN 8      // value dims a lane owns: vdim up to 512
__global__ void __launch_bounds__(MA_WAVES * 64)
masked_attention_kernel(const elem_t* __restrict__ q, const elem_t* __restrict__ cache, const int32_t* __restrict__ block_table,
                        int table_stride, const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_rows,
                        const float* __restrict__ gate, long gate_stride, elem_t* __restrict__ out, int n_tokens, int heads,
                        int kv_heads, int maps, int dim, int vdim, int page_size, int mask_kind, int mask_size, float scale,
                        float softcap, float lambda, float out_scale, float eps, float sink, int gate_per_head) {
  extern __shared__ float smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long item = (long)blockIdx.x * MA_WAVES + wave;
  const bool active = item < (long)n_tokens * heads;
  const int t = active ? (int)(item / heads) : 0, h = active ? (int)(item % heads) : 0;
  const int qw = maps * dim;
  float* qs = smem + (long)wave * qw;
  const elem_t* qsrc = q + ((long)t * heads + h) * qw;
  if (active)
    for (int i = lane; i < qw; i += 64) qs[i] = to_float(qsrc[i]);
  __syncthreads();
  if (!active) return;
  const int g = h / (heads / kv_heads);
  const int kw = kv_heads * maps * dim;
  const long page_elems = (long)page_size * (kw + kv_heads * vdim);
  const int pos = positions[t];
  const int lo = first_seen(pos, mask_kind, mask_size);
  const int32_t* pages = block_table + (long)seq_rows[t] * table_stride;
  float o[MA_OWN];
#pragma unroll
  for (int i = 0; i < MA_OWN; ++i) o[i] = 0.0f;
  for (int mp = 0; mp < maps; ++mp) {
    float acc[MA_OWN];
#pragma unroll
    for (int i = 0; i < MA_OWN; ++i) acc[i] = 0.0f;
    float m = -INFINITY, l = 0.0f;
    const float* qm = qs + mp * dim;
    for (int b = lo / 64; b <= pos / 64; ++b) {
      const int p = b * 64 + lane;
      const bool seen = p >= lo && p <= pos;
      float s = -INFINITY;
      if (seen) {
        const elem_t* key = cache + (long)pages[p / page_size] * page_elems + (long)(p % page_size) * kw + (g * maps + mp) * dim;
        float dot = 0.0f;
        for (int i = 0; i < dim; ++i) dot = fmaf(qm[i], to_float(key[i]), dot);
        s = dot * scale;
        if (softcap > 0.0f) s = softcap * tanhf(s / softcap);
      }
      const float m_new = fmaxf(m, wave_max(s));
      const float w = seen ? expf(s - m_new) : 0.0f;
      const float fold = expf(m - m_new);            // 0 at the first block (m = -inf)
      l = fmaf(l, fold, wave_sum(w));
      m = m_new;
#pragma unroll
      for (int i = 0; i < MA_OWN; ++i) acc[i] *= fold;
      const int j_lo = max(lo, b * 64) - b * 64, j_hi = min(pos, b * 64 + 63) - b * 64;
      for (int j = j_lo; j <= j_hi; ++j) {
        const float wj = __shfl(w, j, 64);
        const int pj = b * 64 + j;
        const elem_t* val = cache + (long)pages[pj / page_size] * page_elems + (long)page_size * kw +
                            (long)g * vdim * page_size + pj % page_size;
#pragma unroll
        for (int i = 0; i < MA_OWN; ++i) {
          const int d = lane + 64 * i;
          if (d < vdim) acc[i] = fmaf(wj, to_float(val[(long)d * page_size]), acc[i]);
        }
      }
    }
    if (sink > -INFINITY) l += expf(sink - m);       // a key of this score that has no value
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < MA_OWN; ++i) o[i] = mp == 0 ? acc[i] * inv : o[i] - lambda * (acc[i] * inv);
  }
  if (maps > 1) {
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < MA_OWN; ++i) ss = fmaf(o[i], o[i], ss);     // dims beyond vdim hold 0
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)vdim + eps);
#pragma unroll
    for (int i = 0; i < MA_OWN; ++i) o[i] = (o[i] * inv) * out_scale;
  }
  elem_t* dst = out + ((long)t * heads + h) * vdim;
#pragma unroll
  for (int i = 0; i < MA_OWN; ++i) {
    const int d = lane + 64 * i;
    if (d >= vdim) continue;
    float v = o[i];
    if (gate != nullptr) v *= 1.0f / (1.0f + expf(-gate[(long)t * gate_stride + (gate_per_head ? (long)h : (long)h * vdim + d)]));
    dst[d] = from_float(v);
  }
}

#if AXON_BF16
typedef __attribute__((ext_vector_type(8))) __bf16 ma_bf16x8;
typedef __attribute__((ext_vector_type(4))) float ma_f32x4;
__device__ inline ma_bf16x8 ma_frag(uint4 v) { return __builtin_bit_cast(ma_bf16x8, v); }

// Operands come from memory or from LDS; an LDS pointer says so in its type, so that its reads are LDS
// instructions with a counter of their own and never wait for the loads from memory that are in flight.
typedef __attribute__((address_space(3))) bf16_t* ma_lds_ptr;
typedef const __attribute__((address_space(3))) bf16_t* ma_lds_cptr;
__device__ inline uint4 ma_load16(const bf16_t* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ inline uint2 ma_load8(const bf16_t* p) { return *reinterpret_cast<const uint2*>(p); }
typedef __attribute__((ext_vector_type(4))) unsigned ma_u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned ma_u32x2;
__device__ inline uint4 ma_load16(ma_lds_cptr p) {
  return __builtin_bit_cast(uint4, *(const __attribute__((address_space(3))) ma_u32x4*)p);
}
__device__ inline uint2 ma_load8(ma_lds_cptr p) {
  return __builtin_bit_cast(uint2, *(const __attribute__((address_space(3))) ma_u32x2*)p);
}
__device__ inline void ma_store16(ma_lds_ptr p, uint4 v) {
  *(__attribute__((address_space(3))) ma_u32x4*)p = __builtin_bit_cast(ma_u32x4, v);
}

// The same attention on the matrix cores: one wave per tile of up to sixteen columns, a block of 64
// positions at a time.  A tile of several tokens (consecutive positions of one request) is those
// tokens for one query head; a tile of one token is that token for up to sixteen query heads of
// one key/value head.  Either way all columns read the same keys and values:
//   S^T [position, column] = K [position, dims] Q^T          (dims in chunks of 32, zero-padded),
//   per column a mask of its own, the bend, a maximum, weights and their sum (a lane holds 16
//   positions of its column; the four lanes of a column meet by lane permutation), the running
//   (m, l) and O^T rescaled, then
//   O^T [dim, column] += V^T [dim, position] P^T             (positions in two chunks of 32),
// with K rows and the rows of V^T as the first operand (16 or 8 bytes a lane) and the rounded
// weights, as they lie in the accumulators, as the second.  Both maps of a differential head run
// side by side over one load of the values; the combination, the norm and the gate happen in
// registers before the store.  DT: tiles of 16 value dims at most; KC: chunks of 32 key dims at
// most.  Pages hold a multiple of 64 positions, dim is a multiple of 8, vdim of 16.
template <int MAPS, int DT>
struct MaState {
  ma_f32x4 acc[MAPS][DT];
  float m[MAPS], l[MAPS];
  __device__ inline void clear() {
#pragma unroll
    for (int mp = 0; mp < MAPS; ++mp) {
      m[mp] = -INFINITY;
      l[mp] = 0.0f;
#pragma unroll
      for (int i = 0; i < DT; ++i) acc[mp][i] = ma_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
  }
};

// One block of 64 positions from p0 for a wave's columns.  kbase: the block's first key row of the
// wave's key/value head, rows kstride apart (a map's keys mp * dim further); vbase: its first value
// row, rows vstride apart, the block's positions side by side; both already moved to the lane's
// slice (8 g, 4 g).  qfrag(mp, c): the lane's query operand of map mp, chunk c.  full: every column
// sees every position of the block (no mask to apply).  The running maximum is kept in units of log2 e.
template <int MAPS, int DT, int KC, class PTR, class QF>
__device__ inline void ma_block(MaState<MAPS, DT>& st, PTR kbase, int kstride, PTR vbase, int vstride,
                                QF qfrag, int p0, int my_lo, int my_pos, bool full, int dim, int dt_n, float scale, float softcap,
                                int j, int g) {
  const int kc = (dim + 31) / 32;
  // the bend's constants: scale 2 log2(e) / c into the exponential; c log2(e) and twice that out of it
  const float bend_in = softcap > 0.0f ? scale * 2.8853900817779268f / softcap : 0.0f, scale_log2 = scale * 1.4426950408889634f;
  const float softcap_log2 = softcap * 1.4426950408889634f, bend_out = 2.0f * softcap_log2;
  uint4 pf[MAPS][2];
  float fold[MAPS];
#pragma unroll
  for (int mp = 0; mp < MAPS; ++mp) {
    ma_f32x4 s[4];
#pragma unroll
    for (int pt = 0; pt < 4; ++pt) {
      s[pt] = ma_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
      const PTR krow = kbase + (16 * pt + j) * kstride + mp * dim;
      uint4 kf[KC];
#pragma unroll
      for (int c = 0; c < KC; ++c)
        if (c < kc) kf[c] = ma_load16(krow + 32 * c);      // beyond dim the query's operand is zero and the row's neighbours are finite
#pragma unroll
      for (int c = 0; c < KC; ++c)
        if (c < kc) s[pt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ma_frag(kf[c]), ma_frag(qfrag(mp, c)), s[pt], 0, 0, 0);
    }
    // scores in units of log2 e, so that a weight is one exp2: s log2(e), bent as c tanh(s / c) =
    // c (1 - 2 / (1 + e^(2 s / c))) where asked
#pragma unroll
    for (int pt = 0; pt < 4; ++pt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v;
        if (softcap > 0.0f) {
          const float e2 = __builtin_amdgcn_exp2f(fminf(s[pt][i] * bend_in, 120.0f));       // e^(2 s / c), kept finite
          v = fmaf(-bend_out, __builtin_amdgcn_rcpf(1.0f + e2), softcap_log2);
        } else {
          v = s[pt][i] * scale_log2;
        }
        s[pt][i] = v;
      }
    if (!full) {
#pragma unroll
      for (int pt = 0; pt < 4; ++pt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int p = p0 + 16 * pt + 4 * g + i;
          s[pt][i] = (p >= my_lo && p <= my_pos) ? s[pt][i] : -INFINITY;
        }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int pt = 0; pt < 4; ++pt)
#pragma unroll
      for (int i = 0; i < 4; ++i) mx = fmaxf(mx, s[pt][i]);
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(st.m[mp], mx);
    const float m_safe = m_new == -INFINITY ? 0.0f : m_new;      // a column that has seen nothing yet
    fold[mp] = __builtin_amdgcn_exp2f(st.m[mp] - m_safe);
    float sum = 0.0f;
#pragma unroll
    for (int pt = 0; pt < 4; ++pt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float w = __builtin_amdgcn_exp2f(s[pt][i] - m_safe);        // 0 where the position is not seen
        s[pt][i] = w;
        sum += w;
      }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    st.l[mp] = fmaf(st.l[mp], fold[mp], sum);
    st.m[mp] = m_new;
#pragma unroll
    for (int c = 0; c < 2; ++c)
      pf[mp][c] = make_uint4(pack2_bf16(s[2 * c][0], s[2 * c][1]), pack2_bf16(s[2 * c][2], s[2 * c][3]),
                             pack2_bf16(s[2 * c + 1][0], s[2 * c + 1][1]), pack2_bf16(s[2 * c + 1][2], s[2 * c + 1][3]));
  }
  constexpr int VB = DT < 4 ? DT : 4;                         // tiles of 16 dims whose rows are asked for together
#pragma unroll
  for (int d0 = 0; d0 < DT; d0 += VB) {
    uint2 v[VB][4];
#pragma unroll
    for (int e = 0; e < VB; ++e) {
      if (d0 + e < dt_n) {
        const PTR vrow = vbase + (16 * (d0 + e) + j) * vstride;
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          v[e][2 * c] = ma_load8(vrow + 32 * c);
          v[e][2 * c + 1] = ma_load8(vrow + 32 * c + 16);
        }
      }
    }
#pragma unroll
    for (int e = 0; e < VB; ++e) {
      if (d0 + e < dt_n) {
#pragma unroll
        for (int mp = 0; mp < MAPS; ++mp) {
          st.acc[mp][d0 + e] *= fold[mp];
#pragma unroll
          for (int c = 0; c < 2; ++c)
            st.acc[mp][d0 + e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                ma_frag(make_uint4(v[e][2 * c].x, v[e][2 * c].y, v[e][2 * c + 1].x, v[e][2 * c + 1].y)), ma_frag(pf[mp][c]),
                st.acc[mp][d0 + e], 0, 0, 0);
        }
      }
    }
  }
}

// A column's outputs (dims 16 dt + 4 g + i in the four lanes j, j + 16, j + 32, j + 48): the maps
// combined, normed, gated and stored.
template <int MAPS, int DT>
__device__ inline void ma_finish(MaState<MAPS, DT>& st, bool my_col, int my_tok, int my_head, int heads, int vdim, int dt_n,
                                 const float* __restrict__ gate, long gate_stride, bf16_t* __restrict__ out, float lambda,
                                 float out_scale, float eps, int g, float sink_log2, int gate_per_head) {
  // the sink: a key of that score (in units of log2 e, like the running maxima) that has no value
  if (sink_log2 > -INFINITY) {
#pragma unroll
    for (int mp = 0; mp < MAPS; ++mp) st.l[mp] += __builtin_amdgcn_exp2f(sink_log2 - st.m[mp]);
  }
  const float inv0 = 1.0f / st.l[0];
  float ss = 0.0f;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
    if (dt < dt_n) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float o = st.acc[0][dt][i] * inv0;
        if (MAPS == 2) {
          o = o - lambda * (st.acc[MAPS - 1][dt][i] * (1.0f / st.l[MAPS - 1]));
          ss = fmaf(o, o, ss);
        }
        st.acc[0][dt][i] = o;
      }
    }
  float norm = 1.0f;
  if (MAPS == 2) {
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    norm = (1.0f / sqrtf(ss / (float)vdim + eps));
  }
  if (!my_col) return;
  bf16_t* dst = out + ((long)my_tok * heads + my_head) * vdim + 4 * g;
  const float* gsrc = gate && !gate_per_head ? gate + (long)my_tok * gate_stride + (long)my_head * vdim + 4 * g : nullptr;
  const float head_gate = gate && gate_per_head ? 1.0f / (1.0f + expf(-gate[(long)my_tok * gate_stride + my_head])) : 1.0f;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
    if (dt < dt_n) {
      float o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        o[i] = st.acc[0][dt][i];
        if (MAPS == 2) o[i] = (o[i] * norm) * out_scale;
        if (gsrc) o[i] *= 1.0f / (1.0f + expf(-gsrc[16 * dt + i]));
        o[i] *= head_gate;
      }
      *reinterpret_cast<uint2*>(dst + 16 * dt) = make_uint2(pack2_bf16(o[0], o[1]), pack2_bf16(o[2], o[3]));
    }
}

// Keys, values and queries straight from memory, a wave a block.  grid (tiles, heads, chunks): with
// `partial` (steps of few single tokens under a window or in chunks) the wave of chunk c takes the
// c-th block of 64 positions of its token alone and leaves (o, m, l) of every column and map,
// unscaled, for the kernel that folds a token's blocks in ascending order; without, it walks them all.
template <int MAPS, int DT, int KC>
__global__ void __launch_bounds__(64)
masked_attention_mfma_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ cache, const int32_t* __restrict__ block_table,
                             int table_stride, const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_rows,
                             const float* __restrict__ gate, long gate_stride, bf16_t* __restrict__ out,
                             const int32_t* __restrict__ tiles, int heads, int kv_heads, int dim, int vdim, int page_size,
                             int mask_kind, int mask_size, float scale, float softcap, float lambda, float out_scale, float eps,
                             float* __restrict__ partial, int n_chunks, float sink_log2, int gate_per_head) {
  constexpr int QMAP = KC * 32, QROW = MAPS * QMAP + 8;      // rows 16 bytes longer than their chunks: 16 rows, 16 banks apart
  __shared__ __align__(16) bf16_t qs[16 * QROW];
  const int lane = threadIdx.x, j = lane & 15, g = lane >> 4;
  const int grp = heads / kv_heads;
  const int t0 = tiles ? tiles[2 * blockIdx.x] : (int)blockIdx.x, n = tiles ? tiles[2 * blockIdx.x + 1] : 1;
  int gk, h0, ncols;
  if (n == 1) {
    const int hc = grp < 16 ? grp : 16, per_kv = (grp + hc - 1) / hc;
    if ((int)blockIdx.y >= kv_heads * per_kv) return;
    gk = blockIdx.y / per_kv;
    const int first = (blockIdx.y % per_kv) * hc;
    h0 = gk * grp + first;
    ncols = min(hc, grp - first);
  } else {
    h0 = blockIdx.y;
    gk = h0 / grp;
    ncols = n;
  }
  const int qw = MAPS * dim;
  for (int idx = lane; idx < 16 * MAPS * KC * 4; idx += 64) {
    const int col = idx / (MAPS * KC * 4), rest = idx % (MAPS * KC * 4), mp = rest / (KC * 4), sl = rest % (KC * 4);
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (col < ncols && 8 * sl < dim) {
      const int tok = n == 1 ? t0 : t0 + col, head = n == 1 ? h0 + col : h0;
      v = *reinterpret_cast<const uint4*>(q + ((long)tok * heads + head) * qw + mp * dim + 8 * sl);
    }
    *reinterpret_cast<uint4*>(qs + col * QROW + mp * QMAP + 8 * sl) = v;
  }
  __syncthreads();
  const int my_tok = n == 1 ? t0 : t0 + j, my_head = n == 1 ? h0 + j : h0;
  const bool my_col = j < ncols;
  const int my_pos = my_col ? positions[my_tok] : -1;
  const int my_lo = my_col ? first_seen(my_pos, mask_kind, mask_size) : 0;
  const int pos_first = positions[t0], pos_last = pos_first + n - 1;
  const int lo_first = first_seen(pos_first, mask_kind, mask_size), lo_last = first_seen(pos_last, mask_kind, mask_size);
  const int32_t* pages = block_table + (long)seq_rows[t0] * table_stride;
  const int kw = kv_heads * MAPS * dim, dt_n = vdim / 16;
  const long page_elems = (long)page_size * (kw + kv_heads * vdim);
  const bf16_t* qlane = qs + j * QROW + 8 * g;
  auto qfrag = [&](int mp, int c) { return *reinterpret_cast<const uint4*>(qlane + mp * QMAP + 32 * c); };
  MaState<MAPS, DT> st;
  st.clear();
  const bool split = partial != nullptr && n == 1;
  if (!split && blockIdx.z > 0) return;
  const int b_first = split ? lo_first / 64 + (int)blockIdx.z : lo_first / 64;
  const int b_last = split ? min(b_first, pos_last / 64) : pos_last / 64;
  for (int b = b_first; b <= b_last; ++b) {
    const int p0 = b * 64, in0 = p0 % page_size;
    const bf16_t* page = cache + (long)pages[p0 / page_size] * page_elems;
    ma_block<MAPS, DT, KC, const bf16_t*>(st, page + (long)in0 * kw + (long)gk * MAPS * dim + 8 * g, kw,
                           page + (long)page_size * kw + (long)gk * vdim * page_size + in0 + 4 * g, page_size, qfrag, p0, my_lo,
                           my_pos, ncols == 16 && p0 >= lo_last && p0 + 63 <= pos_first, dim, dt_n, scale, softcap, j, g);
  }
  if (split) {
    if (!my_col) return;
#pragma unroll
    for (int mp = 0; mp < MAPS; ++mp) {
      float* dst = partial + ((((long)my_tok * heads + my_head) * n_chunks + blockIdx.z) * MAPS + mp) * (vdim + 2);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        if (dt < dt_n) {
#pragma unroll
          for (int i = 0; i < 4; ++i) dst[16 * dt + 4 * g + i] = st.acc[mp][dt][i];
        }
      if (g == 0) {
        dst[vdim] = st.m[mp];
        dst[vdim + 1] = st.l[mp];
      }
    }
    return;
  }
  ma_finish<MAPS, DT>(st, my_col, my_tok, my_head, heads, vdim, dt_n, gate, gate_stride, out, lambda, out_scale, eps, g, sink_log2,
                      gate_per_head);
}

// The blocks of a single token's (head, map) folded in ascending order, a_mp = sum_c e^(m_c - M) o_c /
// sum_c e^(m_c - M) l_c (M the largest m_c; a block that saw nothing has l = 0 and weighs nothing), then
// the maps combined, normed, gated and stored.  One wave per (tile, head); tiles of several tokens were
// finished by the attention kernel itself.
template <int MAPS>
__global__ void __launch_bounds__(64)
masked_attention_fold_kernel(const float* __restrict__ partial, int n_chunks, const int32_t* __restrict__ tiles,
                             const float* __restrict__ gate, long gate_stride, bf16_t* __restrict__ out, int heads, int vdim,
                             float lambda, float out_scale, float eps, float sink_log2, int gate_per_head) {
  const int t = tiles ? tiles[2 * blockIdx.x] : (int)blockIdx.x, n = tiles ? tiles[2 * blockIdx.x + 1] : 1;
  if (n != 1) return;
  const int h = blockIdx.y, lane = threadIdx.x;
  float o[MA_OWN];
#pragma unroll
  for (int i = 0; i < MA_OWN; ++i) o[i] = 0.0f;
  for (int mp = 0; mp < MAPS; ++mp) {
    const float* src = partial + (((long)t * heads + h) * n_chunks * MAPS + mp) * (vdim + 2);
    const long step = (long)MAPS * (vdim + 2);
    // the blocks' (m, l) a lane each, 64 at a time; the largest maximum first, then weights handed round by lane
    float M = -INFINITY;
    for (int c0 = 0; c0 < n_chunks; c0 += 64) {
      const int c = c0 + lane;
      if (c < n_chunks && src[c * step + vdim + 1] > 0.0f) M = fmaxf(M, src[c * step + vdim]);
    }
    M = wave_max(M);
    float L = 0.0f, acc[MA_OWN];
#pragma unroll
    for (int i = 0; i < MA_OWN; ++i) acc[i] = 0.0f;
    for (int c0 = 0; c0 < n_chunks; c0 += 64) {
      const int c = c0 + lane;
      const float lc = c < n_chunks ? src[c * step + vdim + 1] : 0.0f;
      const float w = lc > 0.0f ? exp2f(src[c * step + vdim] - M) : 0.0f;      // the blocks' maxima are in units of log2 e
      L += wave_sum(w * lc);
      // eight blocks' rows asked for together (a row beyond the last is the last again and weighs nothing)
      const int n_here = min(64, n_chunks - c0);
      for (int k0 = 0; k0 < n_here; k0 += 8) {
        float rows[8][MA_OWN];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const float* row = src + (c0 + min(k0 + k, n_here - 1)) * step;
#pragma unroll
          for (int i = 0; i < MA_OWN; ++i) rows[k][i] = row[min(lane + 64 * i, vdim - 1)];
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const float wk = k0 + k < n_here ? __shfl(w, k0 + k, 64) : 0.0f;
#pragma unroll
          for (int i = 0; i < MA_OWN; ++i) acc[i] = fmaf(wk, rows[k][i], acc[i]);
        }
      }
    }
    if (sink_log2 > -INFINITY) L += exp2f(sink_log2 - M);
    const float inv = 1.0f / L;
#pragma unroll
    for (int i = 0; i < MA_OWN; ++i) {
      const float a = lane + 64 * i < vdim ? acc[i] * inv : 0.0f;      // places beyond vdim hold copies: they count as 0
      o[i] = mp == 0 ? a : o[i] - lambda * a;
    }
  }
  if (MAPS > 1) {
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < MA_OWN; ++i) ss = fmaf(o[i], o[i], ss);
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)vdim + eps);
#pragma unroll
    for (int i = 0; i < MA_OWN; ++i) o[i] = (o[i] * inv) * out_scale;
  }
  bf16_t* dst = out + ((long)t * heads + h) * vdim;
#pragma unroll
  for (int i = 0; i < MA_OWN; ++i) {
    const int d = lane + 64 * i;
    if (d >= vdim) continue;
    float v = o[i];
    if (gate != nullptr) v *= 1.0f / (1.0f + expf(-gate[(long)t * gate_stride + (gate_per_head ? (long)h : (long)h * vdim + d)]));
    dst[d] = from_float(v);
  }
}

// Steps with portions of prompts: four waves a block, the four query heads of one key/value head (or as
// many as the group has) on the same tile of tokens.  A block of 64 positions of that head's keys and
// values goes through LDS once for all four (rows 16 bytes longer than their data, against bank
// conflicts), queries wait in registers as operands.  A tile of one token is its first wave's alone
// (up to sixteen heads as columns).
#define MAS_WAVES 4
template <int MAPS, int DT, int KC>
__global__ void __launch_bounds__(MAS_WAVES * 64)
masked_attention_staged_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ cache,
                               const int32_t* __restrict__ block_table, int table_stride, const int32_t* __restrict__ positions,
                               const int32_t* __restrict__ seq_rows, const float* __restrict__ gate, long gate_stride,
                               bf16_t* __restrict__ out, const int32_t* __restrict__ tiles, int heads, int kv_heads, int dim,
                               int vdim, int page_size, int mask_kind, int mask_size, float scale, float softcap, float lambda,
                               float out_scale, float eps, float sink_log2, int gate_per_head) {
  extern __shared__ __align__(16) bf16_t stage[];       // keys [64][MAPS dim + 8], then values [vdim][64 + 8]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, j = lane & 15, g = lane >> 4;
  const int grp = heads / kv_heads, hb_n = (grp + MAS_WAVES - 1) / MAS_WAVES;
  const int t0 = tiles[2 * blockIdx.x], n = tiles[2 * blockIdx.x + 1];
  const int gk = blockIdx.y / hb_n, hb = blockIdx.y % hb_n;
  int h0, ncols;
  bool active;
  if (n == 1) {
    const int hc = grp < 16 ? grp : 16, per_kv = (grp + hc - 1) / hc;
    if (hb >= per_kv) return;                           // the whole block: nothing waits for it
    h0 = gk * grp + hb * hc;
    ncols = min(hc, grp - hb * hc);
    active = wave == 0;
  } else {
    h0 = gk * grp + hb * MAS_WAVES + wave;
    ncols = n;
    active = hb * MAS_WAVES + wave < grp;
  }
  const int my_tok = n == 1 ? t0 : t0 + j, my_head = n == 1 ? h0 + j : h0;
  const bool my_col = active && j < ncols;
  const int qw = MAPS * dim;
  uint4 qf[MAPS][KC];
#pragma unroll
  for (int mp = 0; mp < MAPS; ++mp)
#pragma unroll
    for (int c = 0; c < KC; ++c)
      qf[mp][c] = (my_col && 32 * c + 8 * g < dim)
                      ? *reinterpret_cast<const uint4*>(q + ((long)my_tok * heads + my_head) * qw + mp * dim + 32 * c + 8 * g)
                      : make_uint4(0u, 0u, 0u, 0u);
  auto qfrag = [&](int mp, int c) { return qf[mp][c]; };
  const int my_pos = my_col ? positions[my_tok] : -1;
  const int my_lo = my_col ? first_seen(my_pos, mask_kind, mask_size) : 0;
  const int pos_first = positions[t0], pos_last = pos_first + n - 1;
  const int lo_first = first_seen(pos_first, mask_kind, mask_size), lo_last = first_seen(pos_last, mask_kind, mask_size);
  const int32_t* pages = block_table + (long)seq_rows[t0] * table_stride;
  const int kw = kv_heads * MAPS * dim, dt_n = vdim / 16;
  const long page_elems = (long)page_size * (kw + kv_heads * vdim);
  const int krow = qw + 8, vrow = 64 + 8, k_pieces = qw / 8;
  const ma_lds_ptr ks = (ma_lds_ptr)stage, vs = ks + 64 * krow;
  MaState<MAPS, DT> st;
  st.clear();
  // a block's keys and values travel through registers: asked for while the block before is worked on
  constexpr int KP = MAPS * KC, VP = (DT + 1) / 2;      // 16-byte pieces a thread brings: 64 rows of keys, vdim rows of values
  uint4 kreg[KP], vreg[VP];
  // where a thread's pieces lie in a page and in the stage: the same for every block (-1: none)
  int k_from[KP], k_to[KP], v_from[VP], v_to[VP];
#pragma unroll
  for (int i = 0; i < KP; ++i) {
    const int idx = threadIdx.x + MAS_WAVES * 64 * i, r = idx / k_pieces, piece = idx % k_pieces;
    k_from[i] = idx < 64 * k_pieces ? r * kw + 8 * piece : -1;
    k_to[i] = r * krow + 8 * piece;
  }
#pragma unroll
  for (int i = 0; i < VP; ++i) {
    const int idx = threadIdx.x + MAS_WAVES * 64 * i;
    v_from[i] = idx < vdim * 8 ? (idx >> 3) * page_size + 8 * (idx & 7) : -1;
    v_to[i] = (idx >> 3) * vrow + 8 * (idx & 7);
  }
  auto fetch = [&](int b) {
    const int p0 = b * 64, in0 = p0 % page_size;
    const bf16_t* page = cache + (long)pages[p0 / page_size] * page_elems;
    const bf16_t* ksrc = page + (long)in0 * kw + (long)gk * qw;
    const bf16_t* vsrc = page + (long)page_size * kw + (long)gk * vdim * page_size + in0;
#pragma unroll
    for (int i = 0; i < KP; ++i)
      if (k_from[i] >= 0) kreg[i] = *reinterpret_cast<const uint4*>(ksrc + k_from[i]);
#pragma unroll
    for (int i = 0; i < VP; ++i)
      if (v_from[i] >= 0) vreg[i] = *reinterpret_cast<const uint4*>(vsrc + v_from[i]);
  };
  // the 16 bytes behind each staged key row are read with the last chunk of a map whose dims are no multiple of 32
  // (against a zero query operand): they hold zeros, never what LDS happened to hold
  if (threadIdx.x < 64) ma_store16(ks + threadIdx.x * krow + qw, make_uint4(0u, 0u, 0u, 0u));
  const int b_last = pos_last / 64;
  fetch(lo_first / 64);
  for (int b = lo_first / 64; b <= b_last; ++b) {
    __syncthreads();                                    // the block before has been read
#pragma unroll
    for (int i = 0; i < KP; ++i)
      if (k_from[i] >= 0) ma_store16(ks + k_to[i], kreg[i]);
#pragma unroll
    for (int i = 0; i < VP; ++i)
      if (v_from[i] >= 0) ma_store16(vs + v_to[i], vreg[i]);
    __syncthreads();
    if (b < b_last) fetch(b + 1);
    const int p0 = b * 64;
    if (active)
      ma_block<MAPS, DT, KC, ma_lds_cptr>(st, ks + 8 * g, krow, vs + 4 * g, vrow, qfrag, p0, my_lo, my_pos,
                             ncols == 16 && p0 >= lo_last && p0 + 63 <= pos_first, dim, dt_n, scale, softcap, j, g);
  }
  if (active)
    ma_finish<MAPS, DT>(st, my_col, my_tok, my_head, heads, vdim, dt_n, gate, gate_stride, out, lambda, out_scale, eps, g, sink_log2,
                      gate_per_head);
}

// Blocks of positions a single token can touch under its mask (0: no bound known).  Without a window or chunks
// the bound is the step's: `span`, the positions its longest row sees.
static int masked_chunks(int mask_kind, int mask_size, int span) {
  if (mask_kind == MASK_CAUSAL) return span > 0 ? (span + 63) / 64 : 0;
  return (mask_size + 62) / 64 + 1;
}

template <int MAPS, int DT, int KC>
static int launch_masked_mfma(const void* q, const void* cache, const int32_t* block_table, int table_stride,
                              const int32_t* positions, const int32_t* seq_rows, const float* gate, long gate_stride, void* out,
                              const int32_t* tiles, int n_tiles, int heads, int kv_heads, int dim, int vdim, int page_size,
                              int mask_kind, int mask_size, float scale, float softcap, float lambda, float out_scale, float eps,
                              float* partial, int span, float sink_log2, int gate_per_head, hipStream_t stream) {
  const int grp = heads / kv_heads;
  const size_t lds = ((size_t)64 * (MAPS * dim + 8) + (size_t)vdim * (64 + 8)) * sizeof(bf16_t);
  if (tiles != nullptr && partial == nullptr && KC <= 4 && DT <= 8 && lds <= 64 * 1024) {
    static bool configured = false;
    if (!configured && lds > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&masked_attention_staged_kernel<MAPS, DT, KC>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
      if (e != hipSuccess) {
        axk_set_error("masked_attention: cannot reserve %d bytes of LDS: %s", 64 * 1024, hipGetErrorString(e));
        return -2;
      }
      configured = true;
    }
    masked_attention_staged_kernel<MAPS, DT, KC>
        <<<dim3(n_tiles, kv_heads * ((grp + MAS_WAVES - 1) / MAS_WAVES)), MAS_WAVES * 64, lds, stream>>>(
            (const bf16_t*)q, (const bf16_t*)cache, block_table, table_stride, positions, seq_rows, gate, gate_stride,
            (bf16_t*)out, tiles, heads, kv_heads, dim, vdim, page_size, mask_kind, mask_size, scale, softcap, lambda, out_scale, eps,
            sink_log2, gate_per_head);
    return 0;
  }
  const int n_chunks = partial ? masked_chunks(mask_kind, mask_size, span) : 1;
  masked_attention_mfma_kernel<MAPS, DT, KC><<<dim3(n_tiles, heads, n_chunks), 64, 0, stream>>>(
      (const bf16_t*)q, (const bf16_t*)cache, block_table, table_stride, positions, seq_rows, gate, gate_stride, (bf16_t*)out, tiles,
      heads, kv_heads, dim, vdim, page_size, mask_kind, mask_size, scale, softcap, lambda, out_scale, eps, partial, n_chunks,
      sink_log2, gate_per_head);
  if (partial)
    masked_attention_fold_kernel<MAPS><<<dim3(n_tiles, heads), 64, 0, stream>>>(partial, n_chunks, tiles, gate, gate_stride,
                                                                              (bf16_t*)out, heads, vdim, lambda, out_scale, eps,
                                                                              sink_log2, gate_per_head);
  return 0;
}
#endif

}  // namespace

extern "C" int axk_heads_prepare(const float* proj, long stride, int q_at, int n_q, int k_at, int n_k, int v_at, int v_width,
                                 int dim, const void* q_gain, int q_gain_is_f32, const void* k_gain, int k_gain_is_f32, float eps,
                                 int rot, int neighbours, float magnitude, const float* table, const int32_t* positions,
                                 const int32_t* seq_rows, const int32_t* block_table, int table_stride, void* cache, int page_size,
                                 void* q_out, int n_tokens, int write_kv, float q_temp_coef, int q_temp_every, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && n_q > 0 && n_k > 0 && dim > 0 && v_width > 0 && page_size > 0,
              "heads_prepare: bad sizes T=%d q units=%d k units=%d dim=%d values=%d page=%d", n_tokens, n_q, n_k, dim, v_width,
              page_size);
  AXK_REQUIRE(rot >= 0 && rot <= dim && rot % 2 == 0, "heads_prepare: %d rotated dims of %d", rot, dim);
  AXK_REQUIRE(q_at >= 0 && k_at >= 0 && v_at >= 0 && q_at + (long)n_q * dim <= stride && k_at + (long)n_k * dim <= stride &&
              v_at + (long)v_width <= stride, "heads_prepare: the parts do not fit rows of %ld", stride);
  if (n_tokens == 0) return 0;
  // few tokens: a token's units side by side in several blocks
  const int per_token = n_tokens >= 1024 ? 1 : min((n_q + n_k + 3) / 4, 16);
  heads_prepare_kernel<<<dim3(n_tokens, per_token), 256, 0, (hipStream_t)stream>>>(
      proj, stride, q_at, n_q, k_at, n_k, v_at, v_width, dim, q_gain, q_gain_is_f32, k_gain, k_gain_is_f32, eps, rot, neighbours,
      magnitude, table, positions, seq_rows, block_table, table_stride, (elem_t*)cache, page_size, (elem_t*)q_out, write_kv, q_temp_coef,
      q_temp_every);
  AXK_LAUNCH_CHECK("heads_prepare");
  return 0;
}

// 1 where axk_masked_attention runs on the matrix cores.
extern "C" int axk_masked_attention_uses_mfma(int heads, int kv_heads, int maps, int dim, int vdim, int page_size) {
#if AXON_BF16
  return heads <= 65535 && dim % 8 == 0 && vdim % 16 == 0 && dim <= 256 && vdim <= 256 && page_size % 64 == 0;
#else
  return 0;
#endif
}

// Steps of few tokens: the blocks of 64 positions of a single token run side by side and a second launch folds
// them (under a window or in chunks as many blocks as the mask lets a token touch; else as many as `span`
// positions, what the step's longest row sees, make); the floats of the workspace that takes (0: a wave walks its
// token's blocks itself).
extern "C" long axk_masked_attention_workspace(int n_tokens, int heads, int kv_heads, int maps, int dim, int vdim, int page_size,
                                               int mask_kind, int mask_size, int span) {
#if AXON_BF16
  if (!axk_masked_attention_uses_mfma(heads, kv_heads, maps, dim, vdim, page_size)) return 0;
  const int chunks = masked_chunks(mask_kind, mask_size, span);
  if (chunks < 3 || (long)n_tokens * kv_heads >= 512) return 0;
  return (long)n_tokens * heads * chunks * maps * (vdim + 2);
#else
  return 0;
#endif
}

extern "C" int axk_masked_attention(const void* q, const void* cache, const int32_t* block_table, int table_stride,
                                    const int32_t* positions, const int32_t* seq_rows, const float* gate, long gate_stride,
                                    void* out, int n_tokens, int heads, int kv_heads, int maps, int dim, int vdim, int page_size,
                                    int mask_kind, int mask_size, float scale, float softcap, float lambda, float out_scale,
                                    float eps, const int32_t* tiles, int n_tiles, float* partial, long partial_floats,
                                    float sink, int gate_per_head, int span, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0 && page_size > 0,
              "masked_attention: bad sizes T=%d heads=%d kv heads=%d dim=%d vdim=%d page=%d", n_tokens, heads, kv_heads, dim, vdim,
              page_size);
  AXK_REQUIRE(maps == 1 || maps == 2, "masked_attention: %d score maps a head (1 or 2)", maps);
  AXK_REQUIRE(vdim <= 64 * MA_OWN, "masked_attention: values of %d dims (at most %d)", vdim, 64 * MA_OWN);
  AXK_REQUIRE(mask_kind == MASK_CAUSAL || ((mask_kind == MASK_WINDOW || mask_kind == MASK_CHUNK) && mask_size > 0),
              "masked_attention: mask kind %d of size %d", mask_kind, mask_size);
  AXK_REQUIRE((long)maps * dim * MA_WAVES * 4 <= 64 * 1024, "masked_attention: queries of %d dims do not fit LDS", maps * dim);
  if (n_tokens == 0) return 0;
#if AXON_BF16
  if (axk_masked_attention_uses_mfma(heads, kv_heads, maps, dim, vdim, page_size) && ((uintptr_t)q & 15) == 0 &&
      ((uintptr_t)cache & 15) == 0 && ((uintptr_t)out & 7) == 0) {
    AXK_REQUIRE(tiles == nullptr || n_tiles > 0, "masked_attention: a list of %d tiles", n_tiles);
    const int nt = tiles ? n_tiles : n_tokens;
    const long need = axk_masked_attention_workspace(n_tokens, heads, kv_heads, maps, dim, vdim, page_size, mask_kind, mask_size, span);
    AXK_REQUIRE(partial == nullptr || partial_floats >= need, "masked_attention: a workspace of %ld floats, %ld needed",
                partial_floats, need);
    if (need == 0) partial = nullptr;
#define MA_LAUNCH(MAPS, DT, KC)                                                                                                 \
  rc = launch_masked_mfma<MAPS, DT, KC>(q, cache, block_table, table_stride, positions, seq_rows, gate, gate_stride, out, tiles, nt, \
                                   heads, kv_heads, dim, vdim, page_size, mask_kind, mask_size, scale, softcap, lambda,        \
                                   out_scale, eps, partial, span, sink * 1.4426950408889634f, gate_per_head, (hipStream_t)stream)
    int rc = 0;
    // register tiles by the sizes: chunks of 32 key dims (2, 4 or 8), tiles of 16 value dims (4, 8 or 16)
#define MA_BY_DIM(MAPS, DT)                                                                  \
  {                                                                                          \
    if (dim <= 64) MA_LAUNCH(MAPS, DT, 2); else if (dim <= 128) MA_LAUNCH(MAPS, DT, 4); else MA_LAUNCH(MAPS, DT, 8); \
  }
#define MA_BY_VDIM(MAPS)                                                                     \
  {                                                                                          \
    if (vdim <= 64) MA_BY_DIM(MAPS, 4) else if (vdim <= 128) MA_BY_DIM(MAPS, 8) else MA_BY_DIM(MAPS, 16) \
  }
    if (maps == 1) MA_BY_VDIM(1) else MA_BY_VDIM(2)
#undef MA_BY_VDIM
#undef MA_BY_DIM
#undef MA_LAUNCH
    if (rc != 0) return rc;
    AXK_LAUNCH_CHECK("masked_attention");
    return 0;
  }
#endif
  const long items = (long)n_tokens * heads;
  const size_t lds = (size_t)maps * dim * MA_WAVES * sizeof(float);
  masked_attention_kernel<<<(unsigned)((items + MA_WAVES - 1) / MA_WAVES), MA_WAVES * 64, lds, (hipStream_t)stream>>>(
      (const elem_t*)q, (const elem_t*)cache, block_table, table_stride, positions, seq_rows, gate, gate_stride, (elem_t*)out,
      n_tokens, heads, kv_heads, maps, dim, vdim, page_size, mask_kind, mask_size, scale, softcap, lambda, out_scale, eps, sink,
      gate_per_head);
  AXK_LAUNCH_CHECK("masked_attention");
  return 0;
}
