// A recurrent mixer with a matrix state per head, written by the gated delta rule, and the short
// causal convolution in front of it.
//
//   short_conv        y[t, c] = silu(sum_j w[c, j] * x[t - (taps-1) + j, c]) over the rows of each
//                     request; rows before a portion's first come from the request's tail (its
//                     last taps-1 inputs, kept in its state slot), zeros at a sequence's start.
//   short_conv_tail   the tail after the portion (runs after short_conv: it overwrites what
//                     that one reads).
//   gated_delta       per request and head, token by token (S is dim x vdim, float32):
//                       S <- decay * S;  u = write * (v - S^T k);  S <- S + k u^T;  o = S^T q
//                     with q, k made unit vectors per head first (q also times dim^-1/2),
//                       write = logistic(b),  decay = exp(-exp(A_log) * softplus(a + dt_bias)),
//                     and the read-out o divided by its root mean square over vdim, times a weight
//                     per column and silu(g).
//
// The state of a head lies in memory transposed and padded, [vdim][dim_pad].  Column j of S is
// kept by R neighbouring lanes (4, 8 or 16), each holding a run of its rows: a token costs a lane
// dim/R multiply-adds per pass and the partial sums meet through register moves between the
// lanes, with no barrier inside a tile of tokens.  Columns are independent of one another, so a
// head's work spreads over R * vdim threads however short the step.
// Everything that enters the recurrence is float32 (the projections and the convolution's
// outputs are read in the element type); in the 32-bit engine the scalar gates, the unit norms
// and the read-out's norm are evaluated in 64-bit and rounded once.
#include "common.h"

#include <math.h>

#define DELTA_TILE 16      // tokens whose q, k, gates are prepared together
#define DELTA_MAX_TAPS 16

namespace {

template <typename T>
__global__ __launch_bounds__(256) void short_conv_kernel(
    const T* __restrict__ x, int64_t x_stride, const float* __restrict__ w, const T* __restrict__ tail,
    int64_t tail_stride, const int* __restrict__ cu, const int* __restrict__ slots,
    const int* __restrict__ token_request, T* __restrict__ y, int64_t y_stride, int channels, int taps,
    int num_slots, int row0) {
  const int t = row0 + blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int b = token_request[t];
  const int i = t - cu[b];  // the row's place in its portion
  const int slot = slots[b];
  const T* mine = tail + (int64_t)((slot < 0 || slot >= num_slots) ? num_slots : slot) * tail_stride;
  const float* wc = w + (int64_t)c * taps;
  const int back = taps - 1;
  if constexpr (sizeof(T) == 4) {
    double sum = 0.0;
    for (int j = 0; j < taps; ++j) {
      const int at = i - back + j;  // row of the portion, negative: of the tail
      const float v = at >= 0 ? x[(int64_t)(t - back + j) * x_stride + c] : mine[(int64_t)(back + at) * channels + c];
      sum = fma((double)wc[j], (double)v, sum);
    }
    y[(int64_t)t * y_stride + c] = (float)(sum / (1.0 + exp(-sum)));
  } else {
    float sum = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int at = i - back + j;
      const float v = at >= 0 ? to_f32(x[(int64_t)(t - back + j) * x_stride + c])
                              : to_f32(mine[(int64_t)(back + at) * channels + c]);
      sum = fmaf(wc[j], v, sum);
    }
    y[(int64_t)t * y_stride + c] = from_f32<T>(sum * mi_logistic(sum));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void short_conv_tail_kernel(const T* __restrict__ x, int64_t x_stride,
                                                              T* __restrict__ tail, int64_t tail_stride,
                                                              const int* __restrict__ cu, const int* __restrict__ slots,
                                                              int channels, int taps, int num_slots) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int first = cu[b], n = cu[b + 1] - first;
  if (n <= 0) return;
  const int slot = slots[b];
  T* mine = tail + (int64_t)((slot < 0 || slot >= num_slots) ? num_slots : slot) * tail_stride;
  const int back = taps - 1;
  T old[DELTA_MAX_TAPS];
  for (int j = 0; j < back; ++j) old[j] = mine[(int64_t)j * channels + c];
  for (int j = 0; j < back; ++j) {
    const int at = n - back + j;
    mine[(int64_t)j * channels + c] = at >= 0 ? x[(int64_t)(first + at) * x_stride + c] : old[n + j];
  }
}

// what a token's step needs beside q and k, made once per tile
struct TokenGates {
  float decay, write;
};

// Sum over the R neighbouring lanes that keep one column (R = 4, 8 or 16, inside a row of 16
// lanes); every lane gets the total.  Lane exchanges inside a row are register moves (DPP):
// neighbours, pairs, then the mirror image inside 8 and inside 16 lanes, which after the first
// two steps holds the other half's sum.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int R>
__device__ __forceinline__ float lanes_sum(float v) {
  v += dpp_move<0xB1>(v);  // quad_perm [1,0,3,2]
  v += dpp_move<0x4E>(v);  // quad_perm [2,3,0,1]
  if constexpr (R >= 8) v += dpp_move<0x141>(v);   // row_half_mirror
  if constexpr (R >= 16) v += dpp_move<0x140>(v);  // row_mirror
  return v;
}

// R lanes keep a column of S, lane r of them its rows r * ROWS .. (r + 1) * ROWS - 1 (rows past
// dim are zero and stay zero).  Block: R * vdim threads rounded up to whole waves; thread = R *
// column + r.  The state of a head lies in memory as S transposed and padded, [vdim][R * ROWS].
template <typename T, int R, int ROWS>
__global__ __launch_bounds__(1024) void gated_delta_kernel(
    const T* __restrict__ qkv, int64_t qkv_stride, const T* __restrict__ proj, int64_t proj_stride, int col_b,
    int col_a, int col_g, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
    const float* __restrict__ norm_weight, float* __restrict__ state, int64_t state_stride,
    const int* __restrict__ cu, const int* __restrict__ slots, T* __restrict__ out, int64_t out_stride, int heads,
    int kv_heads, int dim, int vdim, float eps, int num_slots) {
  constexpr bool WIDE = sizeof(T) == 4;
  constexpr int PAD = R * ROWS;  // rows of S as kept: dim rounded up
  extern __shared__ __align__(16) unsigned char lds_bytes[];
  float* q_tile = reinterpret_cast<float*>(lds_bytes);  // [TILE][PAD]
  float* k_tile = q_tile + DELTA_TILE * PAD;            // [TILE][PAD]
  float* o_tile = k_tile + DELTA_TILE * PAD;            // [TILE][vdim]
  TokenGates* gates = reinterpret_cast<TokenGates*>(o_tile + DELTA_TILE * vdim);  // [TILE]

  const int h = blockIdx.x, b = blockIdx.y;
  const int first = cu[b], last = cu[b + 1];
  if (last <= first) return;
  const int slot = slots[b];
  const int tid = threadIdx.x, lane = tid % MI_WAVE, wave = tid / MI_WAVE, n_waves = blockDim.x / MI_WAVE;
  const int j = tid / R, r = tid % R;
  const bool owns = j < vdim;
  const int group = heads / kv_heads;
  const int kvh = h / group;
  float* mine = state + (int64_t)((slot < 0 || slot >= num_slots) ? num_slots : slot) * state_stride +
                ((int64_t)h * vdim + (owns ? j : 0)) * PAD + r * ROWS;
  float s[ROWS];
#pragma unroll
  for (int ii = 0; ii < ROWS; ii += 4) {
    const float4 four = owns ? *reinterpret_cast<const float4*>(mine + ii) : make_float4(0.f, 0.f, 0.f, 0.f);
    s[ii] = four.x, s[ii + 1] = four.y, s[ii + 2] = four.z, s[ii + 3] = four.w;
  }

  const int q_col = kvh * dim, k_col = kv_heads * dim + kvh * dim, v_col = 2 * kv_heads * dim + h * vdim;
  const float rate = expf(a_log[h]);
  const double rate_wide = exp((double)a_log[h]);
  const float q_scale = 1.0f / sqrtf((float)dim);

  for (int t0 = first; t0 < last; t0 += DELTA_TILE) {
    const int nt = min(DELTA_TILE, last - t0);
    __syncthreads();  // the last tile's read-outs have been written out
    // -- q and k of the tile's tokens: unit vectors (float32 from here on); a wave takes a token
    for (int i = wave; i < nt; i += n_waves) {
      const T* row = qkv + (int64_t)(t0 + i) * qkv_stride;
      float qq = 0.f, kk = 0.f;
      double qq_wide = 0.0, kk_wide = 0.0;
      for (int d = lane; d < PAD; d += MI_WAVE) {
        const float qv = d < dim ? to_f32(row[q_col + d]) : 0.f;
        const float kv = d < dim ? to_f32(row[k_col + d]) : 0.f;
        q_tile[i * PAD + d] = qv;
        k_tile[i * PAD + d] = kv;
        if constexpr (WIDE) {
          qq_wide += (double)qv * qv;
          kk_wide += (double)kv * kv;
        } else {
          qq += qv * qv;
          kk += kv * kv;
        }
      }
      float q_inv, k_inv;
      if constexpr (WIDE) {
#pragma unroll
        for (int off = MI_WAVE / 2; off > 0; off >>= 1) {
          qq_wide += __shfl_xor(qq_wide, off, MI_WAVE);
          kk_wide += __shfl_xor(kk_wide, off, MI_WAVE);
        }
        q_inv = (float)(1.0 / sqrt((qq_wide + 1e-6) * (double)dim));
        k_inv = (float)(1.0 / sqrt(kk_wide + 1e-6));
      } else {
        q_inv = rsqrtf(wave_sum(qq) + 1e-6f) * q_scale;
        k_inv = rsqrtf(wave_sum(kk) + 1e-6f);
      }
      for (int d = lane; d < PAD; d += MI_WAVE) {  // (a lane rescales what it wrote itself)
        q_tile[i * PAD + d] *= q_inv;
        k_tile[i * PAD + d] *= k_inv;
      }
      if (lane == 0) {
        const T* p = proj + (int64_t)(t0 + i) * proj_stride;
        const float bv = to_f32(p[col_b + h]), av = to_f32(p[col_a + h]);
        TokenGates gt;
        if constexpr (WIDE) {
          const double z = (double)av + (double)dt_bias[h];
          const double soft = z > 30.0 ? z : log1p(exp(z));
          gt.decay = (float)exp(-rate_wide * soft);
          gt.write = (float)(1.0 / (1.0 + exp(-(double)bv)));
        } else {
          const float z = av + dt_bias[h];
          const float soft = z > 20.f ? z : log1pf(expf(z));
          gt.decay = expf(-rate * soft);
          gt.write = 1.f / (1.f + expf(-bv));
        }
        gates[i] = gt;
      }
    }
    __syncthreads();
    // -- the recurrence over the tile's tokens: no barrier, the lanes of a column meet by register moves
    float v_next = owns ? to_f32(qkv[(int64_t)t0 * qkv_stride + v_col + j]) : 0.f;
    for (int i = 0; i < nt; ++i) {
      const float v = v_next;
      if (i + 1 < nt) v_next = owns ? to_f32(qkv[(int64_t)(t0 + i + 1) * qkv_stride + v_col + j]) : 0.f;
      const TokenGates gt = gates[i];
      const float4* kt = reinterpret_cast<const float4*>(k_tile + i * PAD + r * ROWS);
      const float4* qt = reinterpret_cast<const float4*>(q_tile + i * PAD + r * ROWS);
      float kr[ROWS];
      float seen = 0.f;
#pragma unroll
      for (int ii = 0; ii < ROWS; ii += 4) {
        const float4 four = kt[ii / 4];
        kr[ii] = four.x, kr[ii + 1] = four.y, kr[ii + 2] = four.z, kr[ii + 3] = four.w;
#pragma unroll
        for (int e = 0; e < 4; ++e) seen = fmaf(s[ii + e], kr[ii + e], seen);
      }
      // (S^T k of the decayed state is the decay times S^T k of the old one)
      seen = lanes_sum<R>(seen) * gt.decay;
      const float u = gt.write * (v - seen);
      float read = 0.f;
#pragma unroll
      for (int ii = 0; ii < ROWS; ii += 4) {
        const float4 four = qt[ii / 4];
        const float qr[4] = {four.x, four.y, four.z, four.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          s[ii + e] = fmaf(kr[ii + e], u, s[ii + e] * gt.decay);
          read = fmaf(s[ii + e], qr[e], read);
        }
      }
      read = lanes_sum<R>(read);
      if (owns && r == 0) o_tile[i * vdim + j] = read;
    }
    __syncthreads();
    // -- read-outs of the tile: norm over vdim, weight, gate; a wave takes a token
    for (int i = wave; i < nt; i += n_waves) {
      float sq = 0.f;
      double sq_wide = 0.0;
      for (int d = lane; d < vdim; d += MI_WAVE) {
        const float o = o_tile[i * vdim + d];
        if constexpr (WIDE) sq_wide += (double)o * o;
        else sq += o * o;
      }
      float inv;
      double inv_wide = 0.0;
      if constexpr (WIDE) {
#pragma unroll
        for (int off = MI_WAVE / 2; off > 0; off >>= 1) sq_wide += __shfl_xor(sq_wide, off, MI_WAVE);
        inv_wide = 1.0 / sqrt(sq_wide / (double)vdim + (double)eps);
        inv = (float)inv_wide;
      } else {
        inv = rsqrtf(wave_sum(sq) / (float)vdim + eps);
      }
      const T* p = proj + (int64_t)(t0 + i) * proj_stride + col_g + h * vdim;
      T* dst = out + (int64_t)(t0 + i) * out_stride + h * vdim;
      for (int d = lane; d < vdim; d += MI_WAVE) {
        const float g = to_f32(p[d]);
        if constexpr (WIDE) {
          const double gate = (double)g / (1.0 + exp(-(double)g));
          dst[d] = (float)((double)o_tile[i * vdim + d] * inv_wide * (double)norm_weight[d] * gate);
        } else {
          dst[d] = from_f32<T>(o_tile[i * vdim + d] * inv * norm_weight[d] * (g * mi_logistic(g)));
        }
      }
    }
  }
  if (owns) {
#pragma unroll
    for (int ii = 0; ii < ROWS; ii += 4) *reinterpret_cast<float4*>(mine + ii) = make_float4(s[ii], s[ii + 1], s[ii + 2], s[ii + 3]);
  }
}

// How a head's state is kept for these sizes: R lanes a column (as many as fit a block of 1024
// threads, 16 at most), ROWS rows a lane (4, 16 or 64: the next of them that holds dim / R).
static void delta_layout(int dim, int vdim, int* lanes, int* rows) {
  *lanes = vdim <= 64 ? 16 : (vdim <= 128 ? 8 : 4);
  const int need = ceil_div(dim, *lanes);
  *rows = need <= 4 ? 4 : (need <= 16 ? 16 : 64);
}

}  // namespace

// x: the projections [tokens, >= channels] (row stride); w float32 [channels, taps]; tail
// [slots + 1, (taps-1) * channels] in the element type (row stride); y [tokens, channels].
extern "C" int mi_short_conv(int dtype, const void* x, int64_t x_stride, const float* w, void* tail,
                             int64_t tail_stride, const int* cu, const int* slots, const int* token_request,
                             void* y, int64_t y_stride, int num_tokens, int num_requests, int channels, int taps,
                             int num_slots, hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && num_requests >= 0 && channels > 0, "short_conv: bad sizes tokens=%d requests=%d channels=%d",
             num_tokens, num_requests, channels);
  MI_REQUIRE(taps >= 1 && taps <= DELTA_MAX_TAPS, "short_conv: taps=%d must be 1..%d", taps, DELTA_MAX_TAPS);
  MI_REQUIRE(x_stride >= channels && y_stride >= channels && tail_stride >= (int64_t)(taps - 1) * channels,
             "short_conv: row strides shorter than a row");
  MI_REQUIRE(num_slots >= 1, "short_conv: no state slots");
  MI_REQUIRE(num_requests <= 65535, "short_conv: too many requests");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "short_conv: unknown dtype %d", dtype);
  if (num_tokens == 0 || num_requests == 0) return MI_OK;
  const int blocks = ceil_div(channels, 256);
  for (int first = 0; first < num_tokens; first += 65535) {
    dim3 grid(blocks, min(65535, num_tokens - first));
    if (dtype == MI_F32)
      short_conv_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, x_stride, w, (const float*)tail, tail_stride, cu,
                                                         slots, token_request, (float*)y, y_stride, channels, taps,
                                                         num_slots, first);
    else
      short_conv_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_stride, w, (const bf16_t*)tail, tail_stride,
                                                          cu, slots, token_request, (bf16_t*)y, y_stride, channels, taps,
                                                          num_slots, first);
  }
  MI_CHECK_LAUNCH("short_conv");
  if (taps > 1) {
    dim3 grid(blocks, num_requests);
    if (dtype == MI_F32)
      short_conv_tail_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, x_stride, (float*)tail, tail_stride, cu,
                                                              slots, channels, taps, num_slots);
    else
      short_conv_tail_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_stride, (bf16_t*)tail, tail_stride,
                                                               cu, slots, channels, taps, num_slots);
    MI_CHECK_LAUNCH("short_conv_tail");
  }
  return MI_OK;
}

// qkv: the convolved q | k | v [tokens, 2 * kv_heads * dim + heads * vdim]; proj: the row that
// holds the write gates' (col_b), the decays' (col_a, heads columns each) and the output gates'
// (col_g, heads * vdim columns) projections; state float32 [slots + 1, heads * vdim * dim_pad], dim_pad what
// mi_gated_delta_rows says for these sizes.
extern "C" int mi_gated_delta_rows(int dim, int vdim) {
  int lanes = 0, rows = 0;
  delta_layout(dim, vdim, &lanes, &rows);
  return lanes * rows;
}

extern "C" int mi_gated_delta(int dtype, const void* qkv, int64_t qkv_stride, const void* proj, int64_t proj_stride,
                              int col_b, int col_a, int col_g, const float* a_log, const float* dt_bias,
                              const float* norm_weight, float* state, int64_t state_stride, const int* cu,
                              const int* slots, void* out, int64_t out_stride, int num_requests, int heads,
                              int kv_heads, int dim, int vdim, int dim_pad, float eps, int num_slots, hipStream_t stream) {
  MI_REQUIRE(num_requests >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
             "gated_delta: bad sizes requests=%d heads=%d kv_heads=%d", num_requests, heads, kv_heads);
  MI_REQUIRE(dim > 0 && dim <= 256, "gated_delta: dim=%d must be 1..256", dim);
  MI_REQUIRE(vdim > 0 && vdim <= 256, "gated_delta: vdim=%d must be 1..256", vdim);
  int lanes = 0, rows = 0;
  delta_layout(dim, vdim, &lanes, &rows);
  const int pad = lanes * rows;
  MI_REQUIRE(qkv_stride >= 2 * (int64_t)kv_heads * dim + (int64_t)heads * vdim && out_stride >= (int64_t)heads * vdim,
             "gated_delta: row strides shorter than a row");
  MI_REQUIRE(dim_pad == pad && state_stride >= (int64_t)heads * vdim * pad && state_stride % 4 == 0 &&
                 (uintptr_t)state % 16 == 0,
             "gated_delta: heads of %d x %d keep their state as [vdim][%d] float32 on 16-byte boundaries, the caller has [vdim][%d]",
             dim, vdim, pad, dim_pad);
  MI_REQUIRE(col_b >= 0 && col_a >= 0 && col_g >= 0 && proj_stride >= col_b + heads && proj_stride >= col_a + heads &&
                 proj_stride >= col_g + (int64_t)heads * vdim,
             "gated_delta: the gates' columns lie outside a row of the projections");
  MI_REQUIRE(eps > 0.f, "gated_delta: eps must be positive, got %g", (double)eps);
  MI_REQUIRE(num_slots >= 1 && num_requests <= 65535, "gated_delta: bad slot or request count");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "gated_delta: unknown dtype %d", dtype);
  if (num_requests == 0) return MI_OK;
  const int threads = ceil_div(lanes * vdim, MI_WAVE) * MI_WAVE;
  const size_t lds = sizeof(float) * DELTA_TILE * (2 * pad + vdim) + sizeof(TokenGates) * DELTA_TILE;
  dim3 grid(heads, num_requests);
#define MI_DELTA_LAUNCH(T, RR, ROWS)                                                                                   \
  gated_delta_kernel<T, RR, ROWS><<<grid, threads, lds, stream>>>(                                                     \
      (const T*)qkv, qkv_stride, (const T*)proj, proj_stride, col_b, col_a, col_g, a_log, dt_bias, norm_weight, state, \
      state_stride, cu, slots, (T*)out, out_stride, heads, kv_heads, dim, vdim, eps, num_slots)
#define MI_DELTA_ROWS(T, RR)                      \
  if (rows == 4) MI_DELTA_LAUNCH(T, RR, 4);       \
  else if (rows == 16) MI_DELTA_LAUNCH(T, RR, 16); \
  else MI_DELTA_LAUNCH(T, RR, 64)
#define MI_DELTA_LANES(T)                   \
  if (lanes == 16) { MI_DELTA_ROWS(T, 16); } \
  else if (lanes == 8) { MI_DELTA_ROWS(T, 8); } \
  else { MI_DELTA_ROWS(T, 4); }
  if (dtype == MI_F32) { MI_DELTA_LANES(float) }
  else { MI_DELTA_LANES(bf16_t) }
#undef MI_DELTA_LANES
#undef MI_DELTA_ROWS
#undef MI_DELTA_LAUNCH
  MI_CHECK_LAUNCH("gated_delta");
  return MI_OK;
}
