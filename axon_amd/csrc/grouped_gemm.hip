// Grouped products: many small matrices, each applied to its own rows or its own columns.
//
//   out[orow(r), g ogs + n] = epilogue( sum_k X[xrow(r), g xgs + k] W[g][n][k] + bias[g][n] )
//
// Two ways of saying which rows meet which matrix:
//   * block-diagonal (tiles == null): every row r < M goes through every group g < G, group g
//     reading its own slice of the row's columns (a recurrent layer's gates per block of channels,
//     a per-head projection of an attention layer);
//   * routed (tiles given, on the device): the rows are listed per group in tiles of up to 16
//     (group, first row, count); xrow / orow name the row of X a listed row reads and the row of
//     out it writes (a mixture of experts: rows are (token, chosen expert) pairs in expert order).
//     The grid is launched for the most tiles there can be; blocks beyond *n_tiles leave at once.
//
// Epilogues: bias; a gated linear unit with clamps (W holds 2 N rows a group, gate rows then up
// rows: g = min(gate, limit), u = clamp(up, -limit, limit), out = g sigmoid(alpha g) (u + shift); an
// infinite limit, alpha 1 and shift 0 give silu(gate) up); a multiplication by sigmoid(gate[orow, g ogs + n]),
// or by sigmoid(gate[orow, g]), one number a group; a factor a row on X (row_scale[orow], float32: the sums are
// multiplied by it before bias and unit, as if the row of X had been); out in float32 or in the compute dtype.
//
// The K-reduction of one output is one chain in ascending k that depends on K and the build alone
// (32-bit FMA, or 16x16x32 MFMAs where the bfloat16 build can use them: K a multiple of 32 and
// 16-byte aligned rows), never on which other rows share the tile.
#include "api.h"
#include "common.h"
#include "instances.h"

namespace {

struct GroupedArgs {
  const void* x; int x_is_f32; long x_row_stride; long x_group_stride; const int32_t* x_rows;
  const elem_t* w; const void* bias; int bias_is_f32;
  void* out; int out_is_f32; long out_row_stride; long out_group_stride; const int32_t* out_rows;
  const float* gate; long gate_row_stride; int gate_per_group;
  const float* row_scale;
  int glu; float glu_limit; float glu_alpha; float glu_shift;
  const int32_t* tiles; const int32_t* n_tiles;
  int M, N, K, G;
};

#define GG_ROWS 16
#define GG_COLS 64
#define GG_BK 32

__device__ inline float gg_load_x(const GroupedArgs& a, long at) {
  return a.x_is_f32 ? ((const float*)a.x)[at] : to_float(((const elem_t*)a.x)[at]);
}

__device__ inline float clamped_glu(float gate, float up, float limit, float alpha, float shift) {
  const float g = fminf(gate, limit);
  const float u = fminf(fmaxf(up, -limit), limit);
  return (g * (1.0f / (1.0f + expf(-(alpha * g))))) * (u + shift);
}

__device__ inline void gg_store(const GroupedArgs& a, int g, int orow, int n, float v, float up) {
  if (a.row_scale) {                    // the row of X counts row_scale[orow] times: the product is linear in it
    const float w = a.row_scale[orow];
    v *= w;
    up *= w;
  }
  if (a.bias) {
    const int per = a.glu ? 2 * a.N : a.N;
    v += load_vec(a.bias, a.bias_is_f32, g * per + n);
    if (a.glu) up += load_vec(a.bias, a.bias_is_f32, g * per + a.N + n);
  }
  if (a.glu) v = clamped_glu(v, up, a.glu_limit, a.glu_alpha, a.glu_shift);
  const long col = (long)g * a.out_group_stride + n;
  if (a.gate) v = v * (1.0f / (1.0f + expf(-a.gate[(long)orow * a.gate_row_stride + (a.gate_per_group ? g : col)])));
  const long at = (long)orow * a.out_row_stride + col;
  if (a.out_is_f32) ((float*)a.out)[at] = v;
  else ((elem_t*)a.out)[at] = from_float(v);
}

// which rows and which group this block works on; false: nothing
__device__ inline bool gg_tile(const GroupedArgs& a, int& g, int& first, int& count) {
  if (a.tiles) {
    if ((int)blockIdx.x >= *a.n_tiles) return false;
    g = a.tiles[3 * blockIdx.x];
    first = a.tiles[3 * blockIdx.x + 1];
    count = a.tiles[3 * blockIdx.x + 2];
  } else {
    g = blockIdx.z;
    first = blockIdx.x * GG_ROWS;
    count = min(GG_ROWS, a.M - first);
  }
  return count > 0;
}

// 16 rows x 64 columns at a time in a block of 256 threads: thread (ty, tx) owns rows 4 ty .. 4 ty + 3 of
// column tx.  A listed tile of more than 16 rows (a list made for the tiles of 64) is walked 16 rows at a time.
template <bool GLU>
__global__ void __launch_bounds__(256) grouped_gemm_fma_kernel(GroupedArgs a) {
  __shared__ float xs[GG_ROWS][GG_BK + 1];
  __shared__ float ws[GG_COLS][GG_BK + 1];
  __shared__ float us[GLU ? GG_COLS : 1][GG_BK + 1];
  __shared__ int xrow[GG_ROWS], orow[GG_ROWS];
  int g, tile_first, tile_count;
  if (!gg_tile(a, g, tile_first, tile_count)) return;
  const int tid = threadIdx.x, tx = tid & 63, ty = tid >> 6;
  const int n0 = blockIdx.y * GG_COLS;
  const int w_rows = GLU ? 2 * a.N : a.N;
  const elem_t* wg = a.w + (long)g * w_rows * a.K;
  for (int done = 0; done < tile_count; done += GG_ROWS) {
    const int first = tile_first + done, count = min(GG_ROWS, tile_count - done);
    __syncthreads();
    if (tid < GG_ROWS) {
      const int r = first + min(tid, count - 1);
      xrow[tid] = a.x_rows ? a.x_rows[r] : r;
      orow[tid] = a.out_rows ? a.out_rows[r] : r;
    }
    __syncthreads();
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f}, acc_up[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int k0 = 0; k0 < a.K; k0 += GG_BK) {
      for (int i = tid; i < GG_ROWS * GG_BK; i += 256) {
        const int r = i / GG_BK, kk = i % GG_BK;
        xs[r][kk] = (r < count && k0 + kk < a.K)
                        ? gg_load_x(a, (long)xrow[r] * a.x_row_stride + (long)g * a.x_group_stride + k0 + kk) : 0.0f;
      }
      for (int i = tid; i < GG_COLS * GG_BK; i += 256) {
        const int c = i / GG_BK, kk = i % GG_BK;
        const bool ok = n0 + c < a.N && k0 + kk < a.K;
        ws[c][kk] = ok ? to_float(wg[(long)(n0 + c) * a.K + k0 + kk]) : 0.0f;
        if (GLU) us[c][kk] = ok ? to_float(wg[(long)(a.N + n0 + c) * a.K + k0 + kk]) : 0.0f;
      }
      __syncthreads();
#pragma unroll
      for (int kk = 0; kk < GG_BK; ++kk) {
        const float b = ws[tx][kk];
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = fmaf(xs[ty * 4 + i][kk], b, acc[i]);
        if (GLU) {
          const float bu = us[tx][kk];
#pragma unroll
          for (int i = 0; i < 4; ++i) acc_up[i] = fmaf(xs[ty * 4 + i][kk], bu, acc_up[i]);
        }
      }
      __syncthreads();
    }
    const int n = n0 + tx;
    if (n < a.N) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = ty * 4 + i;
        if (r < count) gg_store(a, g, orow[r], n, acc[i], acc_up[i]);
      }
    }
  }
}

#if AXON_BF16
typedef __attribute__((ext_vector_type(8))) __bf16 gg_bf16x8;
typedef __attribute__((ext_vector_type(4))) float gg_f32x4;

__device__ inline gg_bf16x8 gg_frag(uint4 v) { return __builtin_bit_cast(gg_bf16x8, v); }

__device__ inline uint4 gg_x_frag(const GroupedArgs& a, long at, bool ok) {
  if (!ok) return make_uint4(0, 0, 0, 0);
  if (!a.x_is_f32) return *reinterpret_cast<const uint4*>((const bf16_t*)a.x + at);
  const float4 lo = *reinterpret_cast<const float4*>((const float*)a.x + at);
  const float4 hi = *reinterpret_cast<const float4*>((const float*)a.x + at + 4);
  return make_uint4(pack2_bf16(lo.x, lo.y), pack2_bf16(lo.z, lo.w), pack2_bf16(hi.x, hi.y), pack2_bf16(hi.z, hi.w));
}

// 16 rows x 64 columns a block of four waves, a wave 16 columns: W rows as the MFMA's first
// operand, X rows as its second, both straight from memory (lane l holds row l % 16, the eight k
// from 8 (l / 16)); lane l ends with row l % 16 of the columns 4 (l / 16) .. + 3.  Four steps of
// 32 k are asked for before the first is multiplied.
template <bool GLU>
__global__ void __launch_bounds__(256) grouped_gemm_mfma_kernel(GroupedArgs a) {
  int g, first, count;
  if (!gg_tile(a, g, first, count)) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = blockIdx.y * GG_COLS + wave * 16;
  if (n0 >= a.N) return;
  const int r = lane & 15, kq = (lane >> 4) * 8;
  const bool row_ok = r < count;
  const int rr = first + min(r, count - 1);
  const int xr = a.x_rows ? a.x_rows[rr] : rr;
  const int orow = a.out_rows ? a.out_rows[rr] : rr;
  const long x_at = (long)xr * a.x_row_stride + (long)g * a.x_group_stride + kq;
  const int w_rows = GLU ? 2 * a.N : a.N;
  const bool col_ok = n0 + r < a.N;
  const bf16_t* wrow = a.w + ((long)g * w_rows + min(n0 + r, a.N - 1)) * a.K + kq;
  const bf16_t* urow = wrow + (long)a.N * a.K;
  gg_f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f}, acc_up = {0.0f, 0.0f, 0.0f, 0.0f};
  const uint4 zero = make_uint4(0, 0, 0, 0);
  int k0 = 0;
  for (; k0 + 128 <= a.K; k0 += 128) {
    uint4 xf[4], wf[4], uf[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      xf[s] = gg_x_frag(a, x_at + k0 + 32 * s, row_ok);
      wf[s] = col_ok ? *reinterpret_cast<const uint4*>(wrow + k0 + 32 * s) : zero;
      if (GLU) uf[s] = col_ok ? *reinterpret_cast<const uint4*>(urow + k0 + 32 * s) : zero;
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(gg_frag(wf[s]), gg_frag(xf[s]), acc, 0, 0, 0);
      if (GLU) acc_up = __builtin_amdgcn_mfma_f32_16x16x32_bf16(gg_frag(uf[s]), gg_frag(xf[s]), acc_up, 0, 0, 0);
    }
  }
  for (; k0 < a.K; k0 += 32) {
    const uint4 xf = gg_x_frag(a, x_at + k0, row_ok);
    const uint4 wf = col_ok ? *reinterpret_cast<const uint4*>(wrow + k0) : zero;
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(gg_frag(wf), gg_frag(xf), acc, 0, 0, 0);
    if (GLU) {
      const uint4 uf = col_ok ? *reinterpret_cast<const uint4*>(urow + k0) : zero;
      acc_up = __builtin_amdgcn_mfma_f32_16x16x32_bf16(gg_frag(uf), gg_frag(xf), acc_up, 0, 0, 0);
    }
  }
  if (!row_ok) return;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int n = n0 + (lane >> 4) * 4 + c;
    if (n < a.N) gg_store(a, g, orow, n, acc[c], acc_up[c]);
  }
}
// Many rows a group (a long prompt's pairs of an expert, the tokens of a prompt through a block of
// channels): tiles of 64 rows x 128 rows of W through LDS.  Four waves, two by two, each 32 rows x 64
// rows of W (2 x 4 products a step of 32 k); the next step's operands are asked for while this one is
// multiplied.  With the gated epilogue a block's 128 rows of W are 64 gate rows and the 64 up rows of
// the same columns, and a wave holds both of a column.  The chain of an output is the one of the
// kernel above (16x16x32 products in ascending k), so which of the two runs changes no bit.
#define GT_ROWS 64
#define GT_WROWS 128
template <bool GLU>
__global__ void __launch_bounds__(256) grouped_gemm_tile_kernel(GroupedArgs a) {
  __shared__ __align__(16) bf16_t xs[GT_ROWS * 32];
  __shared__ __align__(16) bf16_t ws[GT_WROWS * 32];
  __shared__ int xrow[GT_ROWS], orow[GT_ROWS];
  int g, first, count;
  if (a.tiles) {
    if ((int)blockIdx.x >= *a.n_tiles) return;
    g = a.tiles[3 * blockIdx.x]; first = a.tiles[3 * blockIdx.x + 1]; count = a.tiles[3 * blockIdx.x + 2];
  } else {
    g = blockIdx.z; first = blockIdx.x * GT_ROWS; count = min(GT_ROWS, a.M - first);
  }
  if (count <= 0) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wr = wave >> 1, wc = wave & 1;
  const int n0 = blockIdx.y * (GLU ? 64 : 128);
  if (tid < GT_ROWS) {
    const int r = first + min(tid, count - 1);
    xrow[tid] = a.x_rows ? a.x_rows[r] : r;
    orow[tid] = a.out_rows ? a.out_rows[r] : r;
  }
  __syncthreads();
  const int w_rows = GLU ? 2 * a.N : a.N;
  const bf16_t* wg = a.w + (long)g * w_rows * a.K;
  // staging: a thread brings 16 bytes of one row of X and of two rows of W a step
  const int srow = tid >> 2, sk = (tid & 3) * 8;
  const bool x_ok = srow < count;
  const long x_at = (long)xrow[srow] * a.x_row_stride + (long)g * a.x_group_stride + sk;
  const bf16_t* wsrc[2];
  bool w_ok[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int slot = srow + 64 * h;
    const int col = GLU ? n0 + srow : n0 + slot;
    w_ok[h] = col < a.N;
    wsrc[h] = wg + (long)((GLU && h) ? a.N + min(col, a.N - 1) : min(col, a.N - 1)) * a.K + sk;
  }
  const uint4 zero = make_uint4(0, 0, 0, 0);
  uint4 px = gg_x_frag(a, x_at, x_ok), pw0 = w_ok[0] ? *reinterpret_cast<const uint4*>(wsrc[0]) : zero,
        pw1 = w_ok[1] ? *reinterpret_cast<const uint4*>(wsrc[1]) : zero;
  gg_f32x4 acc[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = gg_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  const int fr = lane & 15, fk = (lane >> 4) * 8;
  for (int k0 = 0; k0 < a.K; k0 += 32) {
    *reinterpret_cast<uint4*>(&xs[srow * 32 + sk]) = px;
    *reinterpret_cast<uint4*>(&ws[srow * 32 + sk]) = pw0;
    *reinterpret_cast<uint4*>(&ws[(srow + 64) * 32 + sk]) = pw1;
    __syncthreads();
    if (k0 + 32 < a.K) {
      px = gg_x_frag(a, x_at + k0 + 32, x_ok);
      pw0 = w_ok[0] ? *reinterpret_cast<const uint4*>(wsrc[0] + k0 + 32) : zero;
      pw1 = w_ok[1] ? *reinterpret_cast<const uint4*>(wsrc[1] + k0 + 32) : zero;
    }
    uint4 xf[2], wf[4];
#pragma unroll
    for (int i = 0; i < 2; ++i) xf[i] = *reinterpret_cast<const uint4*>(&xs[(32 * wr + 16 * i + fr) * 32 + fk]);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int slot = GLU ? (j < 2 ? 32 * wc + 16 * j : 64 + 32 * wc + 16 * (j - 2)) : 64 * wc + 16 * j;
      wf[j] = *reinterpret_cast<const uint4*>(&ws[(slot + fr) * 32 + fk]);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(gg_frag(wf[j]), gg_frag(xf[i]), acc[i][j], 0, 0, 0);
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = 32 * wr + 16 * i + fr;
    if (r >= count) continue;
#pragma unroll
    for (int j = 0; j < (GLU ? 2 : 4); ++j)
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int n = n0 + (GLU ? 32 * wc + 16 * j : 64 * wc + 16 * j) + (lane >> 4) * 4 + c;
        if (n < a.N) gg_store(a, g, orow[r], n, acc[i][j][c], GLU ? acc[i][j + 2][c] : 0.0f);
      }
  }
}
#endif

}  // namespace

extern "C" int axk_grouped_gemm_uses_mfma(int k, int x_is_f32, long x_row_stride, long x_group_stride) {
#if AXON_BF16
  const int per16 = x_is_f32 ? 4 : 8;     // elements of X in 16 bytes
  return k % 32 == 0 && x_row_stride % per16 == 0 && x_group_stride % per16 == 0;
#else
  return 0;
#endif
}

extern "C" int axk_grouped_gemm(const void* x, int x_is_f32, long x_row_stride, long x_group_stride, const int32_t* x_rows,
                                const void* w, const void* bias, int bias_is_f32, void* out, int out_is_f32,
                                long out_row_stride, long out_group_stride, const int32_t* out_rows, const float* gate,
                                long gate_row_stride, int gate_per_group, const float* row_scale, int glu, float glu_limit,
                                float glu_alpha, float glu_shift, const int32_t* tiles,
                                const int32_t* n_tiles, int max_tiles, int tile_rows, int m, int n, int k, int groups,
                                void* stream) {
  AXK_REQUIRE(m >= 0 && n > 0 && k > 0 && groups > 0, "grouped_gemm: bad sizes M=%d N=%d K=%d groups=%d", m, n, k, groups);
  AXK_REQUIRE((tiles == nullptr) == (n_tiles == nullptr) && (tiles == nullptr || max_tiles >= 0),
              "grouped_gemm: a list of tiles comes with its length and the most tiles there can be");
  AXK_REQUIRE(tiles != nullptr || (x_rows == nullptr && out_rows == nullptr),
              "grouped_gemm: rows are named only beside a list of tiles");
  AXK_REQUIRE(tile_rows == 16 || tile_rows == 64, "grouped_gemm: tiles of %d rows (16 or 64)", tile_rows);
  const int row_tiles = tiles ? max_tiles : ceil_div(m, GG_ROWS);
  if (row_tiles == 0) return 0;
  AXK_REQUIRE(groups <= 65535 && ceil_div(n, GG_COLS) <= 65535, "grouped_gemm: %d groups of %d columns are too many", groups, n);
  GroupedArgs a{x, x_is_f32, x_row_stride, x_group_stride, x_rows, (const elem_t*)w, bias, bias_is_f32, out, out_is_f32,
                out_row_stride, out_group_stride, out_rows, gate, gate_row_stride, gate_per_group, row_scale, glu, glu_limit, glu_alpha,
                glu_shift, tiles, n_tiles,
                m, n, k, groups};
  dim3 grid(row_tiles, ceil_div(n, GG_COLS), tiles ? 1 : groups);
  hipStream_t s = (hipStream_t)stream;
#if AXON_BF16
  const bool mfma = axk_grouped_gemm_uses_mfma(k, x_is_f32, x_row_stride, x_group_stride) && ((uintptr_t)x & 15) == 0 &&
                    ((uintptr_t)w & 15) == 0;
  // many rows a group: tiles of 64 rows through LDS (a list of tiles says by its tile size which it was made for)
  if (mfma && (tiles ? tile_rows == 64 : m >= 256)) {
    dim3 big(tiles ? max_tiles : ceil_div(m, GT_ROWS), ceil_div(n, glu ? 64 : 128), tiles ? 1 : groups);
    if (glu) { AXK_INSTANCE(INST_GROUPED_GEMM, 2, 1); grouped_gemm_tile_kernel<true><<<big, 256, 0, s>>>(a); }
    else { AXK_INSTANCE(INST_GROUPED_GEMM, 2, 0); grouped_gemm_tile_kernel<false><<<big, 256, 0, s>>>(a); }
    AXK_LAUNCH_CHECK("grouped_gemm");
    return 0;
  }
  if (mfma) {
    if (glu) { AXK_INSTANCE(INST_GROUPED_GEMM, 1, 1); grouped_gemm_mfma_kernel<true><<<grid, 256, 0, s>>>(a); }
    else { AXK_INSTANCE(INST_GROUPED_GEMM, 1, 0); grouped_gemm_mfma_kernel<false><<<grid, 256, 0, s>>>(a); }
    AXK_LAUNCH_CHECK("grouped_gemm");
    return 0;
  }
#endif
  if (glu) { AXK_INSTANCE(INST_GROUPED_GEMM, 0, 1); grouped_gemm_fma_kernel<true><<<grid, 256, 0, s>>>(a); }
  else { AXK_INSTANCE(INST_GROUPED_GEMM, 0, 0); grouped_gemm_fma_kernel<false><<<grid, 256, 0, s>>>(a); }
  AXK_LAUNCH_CHECK("grouped_gemm");
  return 0;
}
