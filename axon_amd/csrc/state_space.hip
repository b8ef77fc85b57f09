// A selective state-space mixer in its recurrent form (the "state-space duality" layer of Mamba-2-like
// models): per request and head a state S [N, P] of 32-bit floats, carried from token to token,
//   dt_t = softplus(raw_t + dt_bias),  a_t = exp(-exp(A_log) dt_t),
//   S_t = a_t S_(t-1) + dt_t B_t x_t^T,  y_t = S_t^T C_t + D x_t,
// behind a short causal convolution with silu over the channels [x | B | C], and followed by a gate and
// an RMS norm in equal parts.  Head h reads B and C of group h / (heads / groups).
//
// A request's state row holds two copies of (heads N P floats of S, head by head [N][P], then
// [taps - 1][channels] of the convolution's last inputs, oldest first); zeros for a new request, which
// is also what the convolution reads before the first token.  The state behind position p lives in copy
// p & 1: a step whose first position is s reads copy (s - 1) & 1 and writes the copy of its last
// position, so a step of one token never writes what it read and gives the same state and output if it
// is run again (a decoding step is run once before it is captured into a graph).  The tokens of a
// request are contiguous in a step and a request is in a step once, so two tokens belong to one request
// iff their state slots (seq_rows) are equal.  Everything here is 32-bit in both builds but the
// convolution's weights as stored and the normed output.
#include <math.h>

#include "api.h"
#include "common.h"

namespace {

__device__ inline float ss_silu(float z) { return z / (1.0f + expf(-z)); }
__device__ inline float ss_softplus(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

// u[t, c] = act(bias[c] + sum_k w[c, k] in(t - (taps - 1 - k))) for the channels c of x (float32 rows
// x_stride apart): the last column of w is the current token's; inputs before the step come from the state.
// Threads behind the channels work out the heads' step sizes: terms[t, h] = (dt, a) from raw[t, h].
__global__ void state_conv_kernel(const float* __restrict__ x, long x_stride, const elem_t* __restrict__ w,
                                  const void* __restrict__ bias, int bias_is_f32, int silu, const float* __restrict__ state,
                                  long state_stride, long copy_elems, long tail_at, const int32_t* __restrict__ positions,
                                  const int32_t* __restrict__ seq_rows, float* __restrict__ u, int channels, int taps,
                                  const float* __restrict__ raw, long raw_stride, const void* __restrict__ dt_bias,
                                  int dt_bias_is_f32, const void* __restrict__ a_log, int a_log_is_f32,
                                  float* __restrict__ terms, int heads) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) {
    const int h = c - channels;
    if (h < heads) {
      const float dt = ss_softplus(raw[(long)t * raw_stride + h] + load_vec(dt_bias, dt_bias_is_f32, h));
      terms[((long)t * heads + h) * 2] = dt;
      terms[((long)t * heads + h) * 2 + 1] = expf(-(expf(load_vec(a_log, a_log_is_f32, h)) * dt));
    }
    return;
  }
  const int slot = seq_rows[t];
  // how many earlier tokens of this step belong to the same request (up to taps - 1 matter)
  int inside = 0;
  while (inside < taps - 1 && t - inside - 1 >= 0 && seq_rows[t - inside - 1] == slot) ++inside;
  // the copy behind the position before the request's first of this step
  const int before = (positions[t] - inside + 1) & 1;
  const float* kept = state + (long)slot * state_stride + (long)before * copy_elems + tail_at;      // [taps - 1][channels]
  float acc = 0.0f;
  for (int k = 0; k < taps; ++k) {
    const int back = taps - 1 - k;            // the input `back` tokens before this one
    float v;
    if (back <= inside) v = x[(long)(t - back) * x_stride + c];
    else v = kept[(long)(taps - 1 - (back - inside)) * channels + c];        // the (back - inside)-th last kept input
    acc = fmaf(to_float(w[(long)c * taps + k]), v, acc);
  }
  if (bias) acc += load_vec(bias, bias_is_f32, c);
  u[(long)t * channels + c] = silu ? ss_silu(acc) : acc;
}

// The sum over the sixteen lanes of a row, in every lane of the row, by lane permutations of the adder (pairs,
// quads, halves of the row, the row): a fixed order.
__device__ inline float ss_row_sum(float v) {
#define SS_DPP(val, ctrl) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, val), ctrl, 0xf, 0xf, false))
  v += SS_DPP(v, 0xb1);     // quad_perm [1, 0, 3, 2]
  v += SS_DPP(v, 0x4e);     // quad_perm [2, 3, 0, 1]
  v += SS_DPP(v, 0x141);    // row_half_mirror
  v += SS_DPP(v, 0x140);    // row_mirror
#undef SS_DPP
  return v;
}

// The walk.  grid (requests of the step, heads, blocks of 8 value dims); a block is 128 threads: sixteen
// lanes side by side share a value dim p and hold the state's rows n = lane, lane + 16, ... of that
// column (OWN each: N up to 16 OWN).  The operands of four tokens are asked for while the four before
// them are worked on.  spans [n][3] = (slot, first token, tokens), or null: every token a request of its
// own (a decoding step) in slot seq_rows[t].  u [T, channels] = [x: heads P | B: groups N | C: groups N]
// behind the convolution; terms [T, heads, 2] = (dt, a).  y [T, heads P] float32.  The block (head 0,
// dims 0) also brings the convolution's kept inputs up to date from conv_in (the convolution's inputs,
// float32 rows conv_in_stride apart).  A sum over n is sixteen partial chains in ascending n folded in a
// fixed order: the same for a token however the request was cut into steps.  FULL: N is 16 OWN, so no row
// of a lane lies beyond the state (a lane's rows of B and C are then one address and constant offsets, and
// nothing has to be kept at zero: a wave of this kernel is bound by the instructions it issues a token).
#define SS_AHEAD 4
#define SS_THREADS 128
template <int OWN>
struct SsOperands {
  float x[SS_AHEAD], dt[SS_AHEAD], a[SS_AHEAD], B[SS_AHEAD][OWN], C[SS_AHEAD][OWN];
};

template <int OWN, bool FULL>
__global__ void __launch_bounds__(SS_THREADS)
state_space_scan_kernel(const float* __restrict__ u, const float* __restrict__ terms, const void* __restrict__ d_skip,
                        int d_is_f32, float* __restrict__ state, long state_stride, long copy_elems, long tail_at,
                        const int32_t* __restrict__ spans, const int32_t* __restrict__ positions,
                        const int32_t* __restrict__ seq_rows, const float* __restrict__ conv_in, long conv_in_stride,
                        float* __restrict__ y, int heads, int groups, int P, int N, int channels, int taps,
                        const int32_t* __restrict__ segs, float* __restrict__ ends, float* __restrict__ cum) {
  int slot, first, count;
  bool from_state = true;
  if (segs) {
    slot = segs[4 * blockIdx.x]; first = segs[4 * blockIdx.x + 1]; count = segs[4 * blockIdx.x + 2];
    from_state = segs[4 * blockIdx.x + 3] != 0;
  } else if (spans) {
    slot = spans[3 * blockIdx.x]; first = spans[3 * blockIdx.x + 1]; count = spans[3 * blockIdx.x + 2];
  } else {
    slot = seq_rows[blockIdx.x]; first = blockIdx.x; count = 1;
  }
  const int h = blockIdx.y, g = h / (heads / groups);
  const int ns = threadIdx.x & 15, p = blockIdx.z * (SS_THREADS / 16) + (threadIdx.x >> 4);
  const bool has_p = p < P;
  const int start = positions[first];
  const float* from = state + (long)slot * state_stride + (long)((start + 1) & 1) * copy_elems;
  float* to = state + (long)slot * state_stride + (long)((start + count - 1) & 1) * copy_elems;
  const int inner = heads * P;
  const long s_at = (long)h * N * P;
  float S[OWN];
  int n_of[OWN];
#pragma unroll
  for (int i = 0; i < OWN; ++i) {
    const int n = ns + 16 * i;
    S[i] = from_state && has_p && n < N ? from[s_at + (long)n * P + p] : 0.0f;
    n_of[i] = min(n, N - 1);            // rows beyond N hold zeros in S: what they meet does not count
  }
  const float dskip = load_vec(d_skip, d_is_f32, h);
  const long x_col = (long)h * P + (has_p ? p : 0), b_col = inner + (long)g * N, c_col = inner + (long)groups * N + (long)g * N;
  const int last = first + count;
  const long lane_b = b_col + ns, lane_c = c_col + ns;
  auto fetch = [&](SsOperands<OWN>& o, int t0) {
#pragma unroll
    for (int k = 0; k < SS_AHEAD; ++k) {
      const int t = min(t0 + k, last - 1);             // behind the last token: the last again, not used
      const float* row = u + (long)t * channels;
      const float* bp = row + lane_b;
      const float* cp = row + lane_c;
      o.x[k] = row[x_col];
      o.dt[k] = terms[((long)t * heads + h) * 2];
      o.a[k] = terms[((long)t * heads + h) * 2 + 1];
#pragma unroll
      for (int i = 0; i < OWN; ++i) {
        o.B[k][i] = FULL ? bp[16 * i] : row[b_col + n_of[i]];
        o.C[k][i] = FULL ? cp[16 * i] : row[c_col + n_of[i]];
      }
    }
  };
  float decay = 1.0f;                  // of a segment: the product of its tokens' a so far
  const bool tells_decay = cum != nullptr && blockIdx.z == 0 && threadIdx.x == 0;
  auto work = [&](const SsOperands<OWN>& o, int t0) {
#pragma unroll
    for (int k = 0; k < SS_AHEAD; ++k) {
      if (t0 + k < last) {
        decay *= o.a[k];
        if (tells_decay) cum[(long)(t0 + k) * heads + h] = decay;
        const float dx = o.dt[k] * o.x[k];
        float part = 0.0f;
#pragma unroll
        for (int i = 0; i < OWN; ++i) {
          S[i] = FULL || ns + 16 * i < N ? fmaf(o.a[k], S[i], dx * o.B[k][i]) : 0.0f;
          part = fmaf(S[i], o.C[k][i], part);
        }
        part = ss_row_sum(part);
        if (ns == 0 && has_p) y[(long)(t0 + k) * inner + x_col] = fmaf(dskip, o.x[k], part);
      }
    }
  };
  SsOperands<OWN> even, odd;
  fetch(even, first);
  for (int t = first; t < last; t += 2 * SS_AHEAD) {
    if (t + SS_AHEAD < last) fetch(odd, t + SS_AHEAD);
    work(even, t);
    if (t + SS_AHEAD >= last) break;
    if (t + 2 * SS_AHEAD < last) fetch(even, t + 2 * SS_AHEAD);
    work(odd, t + SS_AHEAD);
  }
  if (segs) {                          // a segment's end state goes to the workspace; the fold brings the request's state up to date
    float* end = ends + ((long)blockIdx.x * heads + h) * N * P;
#pragma unroll
    for (int i = 0; i < OWN; ++i) {
      const int n = ns + 16 * i;
      if (has_p && n < N) end[(long)n * P + p] = S[i];
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < OWN; ++i) {
    const int n = ns + 16 * i;
    if (has_p && n < N) to[s_at + (long)n * P + p] = S[i];
  }
  if (blockIdx.y != 0 || blockIdx.z != 0) return;
  // the convolution's last taps - 1 inputs: of (what was kept, this step's inputs) the last taps - 1; place
  // i takes what lies `count` places later (where both copies are one: read before it is written, ascending)
  float* kept = to + tail_at;
  const float* kept_from = from + tail_at;
  for (int c = threadIdx.x; c < channels; c += blockDim.x)
    for (int i = 0; i < taps - 1; ++i) {
      const int at = i + count;
      kept[(long)i * channels + c] = at < taps - 1 ? kept_from[(long)at * channels + c]
                                                   : conv_in[(long)(first + at - (taps - 1)) * conv_in_stride + c];
    }
}

// Long stretches of tokens in segments.  The scan above then runs every segment of a request side by side:
// the first from the request's state, the others from zero, each leaving its end state E_k in `ends` and
// the running product of its tokens' a in `cum`.  Two more launches make the rest:
//   the fold, per (request, head, eight value dims), over the request's segments in order: the state a
//   segment starts from is I_1 = E_0, I_(k+1) = D_k I_k + E_k (D_k: the segment's whole product), left in
//   `ends` in E_k's place; the last one is the request's new state (and the block (head 0, dims 0) brings
//   the convolution's kept inputs up to date);
//   the carry, per (segment but the first, head, eight value dims): y_t += cum_t (I_k^T C_t), what the
//   state the segment did not start from adds to its outputs; tokens are independent here.
// The sums of a token then differ in order from the walk of one chain, by rounding, and which tokens share a
// segment goes by how the request was cut into steps.
// spans5 [n][5] = (slot, first token, tokens, first segment, segments).
#define SS_CARRY 32        // tokens of a segment a block of the carry takes
template <int OWN>
__global__ void __launch_bounds__(SS_THREADS)
state_space_fold_kernel(float* __restrict__ ends, const float* __restrict__ cum, const int32_t* __restrict__ spans5,
                        const int32_t* __restrict__ segs, float* __restrict__ state, long state_stride, long copy_elems,
                        long tail_at, const int32_t* __restrict__ positions, const float* __restrict__ conv_in,
                        long conv_in_stride, int heads, int P, int N, int channels, int taps) {
  const int slot = spans5[5 * blockIdx.x], first = spans5[5 * blockIdx.x + 1], count = spans5[5 * blockIdx.x + 2];
  const int seg0 = spans5[5 * blockIdx.x + 3], n_segs = spans5[5 * blockIdx.x + 4];
  const int h = blockIdx.y;
  const int ns = threadIdx.x & 15, p = blockIdx.z * (SS_THREADS / 16) + (threadIdx.x >> 4);
  const bool has_p = p < P;
  const int start = positions[first];
  const float* from = state + (long)slot * state_stride + (long)((start + 1) & 1) * copy_elems;
  float* to = state + (long)slot * state_stride + (long)((start + count - 1) & 1) * copy_elems;
  float I[OWN];
#pragma unroll
  for (int i = 0; i < OWN; ++i) {
    const int n = ns + 16 * i;
    I[i] = has_p && n < N ? ends[((long)seg0 * heads + h) * N * P + (long)n * P + p] : 0.0f;
  }
  for (int k = 1; k < n_segs; ++k) {
    const int seg = seg0 + k;
    const int seg_last = segs[4 * seg + 1] + segs[4 * seg + 2] - 1;
    const float D = cum[(long)seg_last * heads + h];
    float* E = ends + ((long)seg * heads + h) * N * P;
#pragma unroll
    for (int i = 0; i < OWN; ++i) {
      const int n = ns + 16 * i;
      if (has_p && n < N) {
        const float e = E[(long)n * P + p];
        E[(long)n * P + p] = I[i];
        I[i] = fmaf(D, I[i], e);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < OWN; ++i) {
    const int n = ns + 16 * i;
    if (has_p && n < N) to[(long)h * N * P + (long)n * P + p] = I[i];
  }
  if (blockIdx.y != 0 || blockIdx.z != 0) return;
  float* kept = to + tail_at;
  const float* kept_from = from + tail_at;
  for (int c = threadIdx.x; c < channels; c += blockDim.x)
    for (int i = 0; i < taps - 1; ++i) {
      const int at = i + count;
      kept[(long)i * channels + c] = at < taps - 1 ? kept_from[(long)at * channels + c]
                                                   : conv_in[(long)(first + at - (taps - 1)) * conv_in_stride + c];
    }
}

template <int OWN>
__global__ void __launch_bounds__(SS_THREADS)
state_space_carry_kernel(const float* __restrict__ u, const float* __restrict__ ends, const float* __restrict__ cum,
                         const int32_t* __restrict__ segs, float* __restrict__ y, int heads, int groups, int P, int N,
                         int channels, int pieces) {
  // blockIdx.x: (segment, piece of SS_CARRY tokens of it); tokens are independent here
  const int seg = blockIdx.x / pieces, piece = blockIdx.x % pieces;
  if (segs[4 * seg + 3] != 0) return;                 // a request's first segment started from its state
  const int seg_first = segs[4 * seg + 1], seg_count = segs[4 * seg + 2];
  if (piece * SS_CARRY >= seg_count) return;
  const int first = seg_first + piece * SS_CARRY, count = min(SS_CARRY, seg_count - piece * SS_CARRY);
  const int h = blockIdx.y, g = h / (heads / groups);
  const int ns = threadIdx.x & 15, p = blockIdx.z * (SS_THREADS / 16) + (threadIdx.x >> 4);
  const bool has_p = p < P;
  const int inner = heads * P;
  const float* carried = ends + ((long)seg * heads + h) * N * P;
  float I[OWN];
  int n_of[OWN];
#pragma unroll
  for (int i = 0; i < OWN; ++i) {
    const int n = ns + 16 * i;
    I[i] = has_p && n < N ? carried[(long)n * P + p] : 0.0f;
    n_of[i] = min(n, N - 1);
  }
  const long c_col = inner + (long)groups * N + (long)g * N;
  const long out_col = (long)h * P + (has_p ? p : 0);
  for (int t0 = first; t0 < first + count; t0 += SS_AHEAD) {
    float C[SS_AHEAD][OWN], c[SS_AHEAD], was[SS_AHEAD];
#pragma unroll
    for (int k = 0; k < SS_AHEAD; ++k) {
      const int t = min(t0 + k, first + count - 1);
      const float* row = u + (long)t * channels + c_col;
#pragma unroll
      for (int i = 0; i < OWN; ++i) C[k][i] = row[n_of[i]];
      c[k] = cum[(long)t * heads + h];
      was[k] = y[(long)t * inner + out_col];
    }
#pragma unroll
    for (int k = 0; k < SS_AHEAD; ++k) {
      float part = 0.0f;
#pragma unroll
      for (int i = 0; i < OWN; ++i) part = fmaf(I[i], C[k][i], part);
      part = ss_row_sum(part);
      if (t0 + k < first + count && ns == 0 && has_p) y[(long)(t0 + k) * inner + out_col] = fmaf(c[k], part, was[k]);
    }
  }
}

// out[t, part] = ((v / sqrt(mean(v^2) + eps)) gain) with v = y[t, part] silu(z[t, part]): the gate first,
// then the norm of each of `parts` equal parts of a row by its own root mean square.  A block a (token, part):
// a strided chain a thread, a butterfly a wave, the four waves in order.
__global__ void __launch_bounds__(256)
gated_group_norm_kernel(const float* __restrict__ y, const float* __restrict__ z, long z_stride, const void* __restrict__ gain,
                        int gain_is_f32, float eps, elem_t* __restrict__ out, int width, int parts) {
  __shared__ float partial[256 / AXON_WAVE];
  const int t = blockIdx.x / parts, part = blockIdx.x % parts, size = width / parts;
  const float* ys = y + (long)t * width + (long)part * size;
  const float* zs = z + (long)t * z_stride + (long)part * size;
  float kept[4];                      // parts of up to 1,024 values are read once
  float ss = 0.0f;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int i = threadIdx.x + 256 * c;
    kept[c] = i < size ? ys[i] * ss_silu(zs[i]) : 0.0f;
    ss = fmaf(kept[c], kept[c], ss);
  }
  for (int i = threadIdx.x + 1024; i < size; i += 256) {
    const float v = ys[i] * ss_silu(zs[i]);
    ss = fmaf(v, v, ss);
  }
  const float inv = 1.0f / sqrtf(block_sum_256(ss, partial) / (float)size + eps);
  elem_t* dst = out + (long)t * width + (long)part * size;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int i = threadIdx.x + 256 * c;
    if (i < size) dst[i] = from_float((kept[c] * inv) * load_vec(gain, gain_is_f32, part * size + i));
  }
  for (int i = threadIdx.x + 1024; i < size; i += 256) {
    const float v = ys[i] * ss_silu(zs[i]);
    dst[i] = from_float((v * inv) * load_vec(gain, gain_is_f32, part * size + i));
  }
}

}  // namespace

extern "C" int axk_state_conv(const float* x, long x_stride, const void* w, const void* bias, int bias_is_f32, int silu,
                              const float* state, long state_stride, long copy_elems, long tail_at, const int32_t* positions,
                              const int32_t* seq_rows, float* u, int n_tokens, int channels, int taps, const float* raw,
                              long raw_stride, const void* dt_bias, int dt_bias_is_f32, const void* a_log, int a_log_is_f32,
                              float* terms, int heads, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && channels > 0 && taps >= 1 && x_stride >= channels && heads >= 0,
              "state_conv: bad sizes T=%d channels=%d taps=%d heads=%d row stride %ld", n_tokens, channels, taps, heads, x_stride);
  AXK_REQUIRE(tail_at >= 0 && copy_elems >= tail_at + (long)(taps - 1) * channels && state_stride >= 2 * copy_elems,
              "state_conv: a state row of %ld floats does not hold two copies of %ld with %d x %d kept inputs from %ld",
              state_stride, copy_elems, taps - 1, channels, tail_at);
  AXK_REQUIRE(heads == 0 || (raw != nullptr && dt_bias != nullptr && a_log != nullptr && terms != nullptr && raw_stride >= heads),
              "state_conv: step sizes of %d heads need their inputs", heads);
  AXK_REQUIRE(n_tokens <= 65535, "state_conv: %d tokens in one step (at most 65535)", n_tokens);
  if (n_tokens == 0) return 0;
  dim3 grid(ceil_div(channels + heads, 256), n_tokens);
  state_conv_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(x, x_stride, (const elem_t*)w, bias, bias_is_f32, silu, state,
                                                          state_stride, copy_elems, tail_at, positions, seq_rows, u, channels,
                                                          taps, raw, raw_stride, dt_bias, dt_bias_is_f32, a_log, a_log_is_f32,
                                                          terms, heads);
  AXK_LAUNCH_CHECK("state_conv");
  return 0;
}

extern "C" int axk_state_space_scan(const float* u, const float* terms, const void* d_skip, int d_is_f32, float* state,
                                    long state_stride, long copy_elems, long tail_at, const int32_t* spans, int n_spans,
                                    const int32_t* positions, const int32_t* seq_rows, const float* conv_in, long conv_in_stride,
                                    float* y, int heads, int groups, int vdim, int n_state, int taps, const int32_t* segs,
                                    int n_segs, int longest_seg, const int32_t* spans5, float* ends, float* cum, void* stream) {
  AXK_REQUIRE(n_spans >= 0 && heads > 0 && groups > 0 && heads % groups == 0 && vdim > 0 && n_state > 0 && taps >= 1,
              "state_space_scan: bad sizes spans=%d heads=%d groups=%d vdim=%d state=%d taps=%d", n_spans, heads, groups, vdim,
              n_state, taps);
  AXK_REQUIRE(n_state <= 256, "state_space_scan: a state of %d rows a head (at most 256)", n_state);
  const int channels = heads * vdim + 2 * groups * n_state;
  AXK_REQUIRE(tail_at >= (long)heads * n_state * vdim && copy_elems >= tail_at + (long)(taps - 1) * channels &&
              state_stride >= 2 * copy_elems && conv_in_stride >= channels,
              "state_space_scan: a state row of %ld floats does not hold two copies of %ld (%d x %d x %d, then %d x %d from %ld)",
              state_stride, copy_elems, heads, n_state, vdim, taps - 1, channels, tail_at);
  AXK_REQUIRE((spans != nullptr || seq_rows != nullptr) && positions != nullptr, "state_space_scan: neither spans nor slots, or no positions");
  AXK_REQUIRE(n_spans <= 65535 * 32 && heads <= 65535 && ceil_div(vdim, SS_THREADS / 16) <= 65535, "state_space_scan: %d requests of %d heads", n_spans, heads);
  if (n_spans == 0) return 0;
  AXK_REQUIRE(segs == nullptr || (n_segs >= n_spans && spans5 != nullptr && ends != nullptr && cum != nullptr && spans != nullptr),
              "state_space_scan: %d segments of %d requests come with the requests' list, a workspace and the running products",
              n_segs, n_spans);
  dim3 grid(segs ? n_segs : n_spans, heads, ceil_div(vdim, SS_THREADS / 16));
  dim3 grid_fold(n_spans, heads, ceil_div(vdim, SS_THREADS / 16));
  AXK_REQUIRE(segs == nullptr || longest_seg > 0, "state_space_scan: segments of at most %d tokens", longest_seg);
  const int pieces = segs ? ceil_div(longest_seg, SS_CARRY) : 1;
  dim3 grid_carry((unsigned)((long)(segs ? n_segs : 1) * pieces), heads, ceil_div(vdim, SS_THREADS / 16));
  hipStream_t s = (hipStream_t)stream;
#define SS_ARGS u, terms, d_skip, d_is_f32, state, state_stride, copy_elems, tail_at, spans, positions, seq_rows, conv_in, conv_in_stride, y, \
                heads, groups, vdim, n_state, channels, taps, segs, ends, cum
#define SS_LAUNCH(OWN)                                                                              \
  {                                                                                                 \
    if (n_state == 16 * OWN) state_space_scan_kernel<OWN, true><<<grid, SS_THREADS, 0, s>>>(SS_ARGS); \
    else state_space_scan_kernel<OWN, false><<<grid, SS_THREADS, 0, s>>>(SS_ARGS);                  \
    if (segs) {                                                                                     \
      state_space_fold_kernel<OWN><<<grid_fold, SS_THREADS, 0, s>>>(ends, cum, spans5, segs, state, state_stride, copy_elems, tail_at, \
                                                                    positions, conv_in, conv_in_stride, heads, vdim, n_state, channels, taps); \
      state_space_carry_kernel<OWN><<<grid_carry, SS_THREADS, 0, s>>>(u, ends, cum, segs, y, heads, groups, vdim, n_state, channels, pieces); \
    }                                                                                               \
  }
  if (n_state <= 16) SS_LAUNCH(1)
  else if (n_state <= 32) SS_LAUNCH(2)
  else if (n_state <= 64) SS_LAUNCH(4)
  else if (n_state <= 128) SS_LAUNCH(8)
  else SS_LAUNCH(16)
#undef SS_LAUNCH
#undef SS_ARGS
  AXK_LAUNCH_CHECK("state_space_scan");
  return 0;
}

extern "C" int axk_gated_group_norm(const float* y, const float* z, long z_stride, const void* gain, int gain_is_f32, float eps,
                                    void* out, int n_tokens, int width, int parts, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && width > 0 && parts > 0 && width % parts == 0 && z_stride >= width,
              "gated_group_norm: bad sizes T=%d width=%d parts=%d", n_tokens, width, parts);
  if (n_tokens == 0) return 0;
  AXK_REQUIRE((long)n_tokens * parts <= 2147483647L, "gated_group_norm: %d tokens in %d parts", n_tokens, parts);
  gated_group_norm_kernel<<<(unsigned)((long)n_tokens * parts), 256, 0, (hipStream_t)stream>>>(y, z, z_stride, gain, gain_is_f32, eps,
                                                                                               (elem_t*)out, width, parts);
  AXK_LAUNCH_CHECK("gated_group_norm");
  return 0;
}
