// Kernels of a layer whose sublayers all read one norm of the stream and whose outputs are
// added to the stream together, and of the clamped gated feed-forward.
//
//   stream_update_norm   x += scale * (a + b + bias) + shift   (float32 stream, in place),
//                        then RMS norm of the new rows times a weight -> compute dtype.
//                        Any of a, b, bias, shift may be absent; so may the norm.  One launch
//                        stands between two layers: the add that ends one and the norm that
//                        begins the next.
//   clamped_glu          [gate | up] + biases -> min(gate, limit) * logistic(slope * gate') *
//                        (clamp(up, -limit, limit) + 1), gate' the clamped gate.
//
// float32 elements (the 32-bit engine): statistics and activations are evaluated in 64-bit
// and rounded once, as everywhere in this library.
#include "common.h"

#include <math.h>

namespace {

__device__ __forceinline__ double wave_sum_wide(double v) {
#pragma unroll
  for (int off = MI_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, MI_WAVE);
  return v;
}

__device__ __forceinline__ double block_sum_wide(double v, double* scratch) {
  v = wave_sum_wide(v);
  const int wave = threadIdx.x / MI_WAVE, lane = threadIdx.x % MI_WAVE;
  const int n_waves = (blockDim.x + MI_WAVE - 1) / MI_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  double total = 0.0;
  for (int w = 0; w < n_waves; ++w) total += scratch[w];
  return total;
}

// One block a row.  `rows` (optional) lists the rows to norm; with it the stream is left as
// it was (the rows' new values are used for the norm only), as the final norm wants it.
template <typename T>
__global__ __launch_bounds__(1024) void stream_update_norm_kernel(
    const T* __restrict__ a, int64_t a_stride, const T* __restrict__ b, int64_t b_stride,
    const float* __restrict__ bias, const float* __restrict__ shift, float scale, float* __restrict__ stream,
    const T* __restrict__ weight, T* __restrict__ out, const int* __restrict__ rows, int hidden, float eps) {
  __shared__ float scratch[16];
  __shared__ double scratch_wide[16];
  constexpr bool WIDE = sizeof(T) == 4;
  const int r = blockIdx.x;
  const int t = rows ? rows[r] : r;
  float* x = stream + (int64_t)t * hidden;
  const T* ar = a ? a + (int64_t)t * a_stride : nullptr;
  const T* br = b ? b + (int64_t)t * b_stride : nullptr;
  // a thread keeps its columns' new values (up to 8 of them; wider rows are read again)
  constexpr int KEEP = 8;
  float kept[KEEP];
  float squares = 0.f;
  double squares_wide = 0.0;
  int n = 0;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x, ++n) {
    float value;
    if constexpr (WIDE) {
      double sum = 0.0;
      if (ar) sum += (double)ar[c];
      if (br) sum += (double)br[c];
      if (bias) sum += (double)bias[c];
      double v = (double)x[c] + (double)scale * sum;
      if (shift) v += (double)shift[c];
      value = (float)v;
      squares_wide += (double)value * (double)value;
    } else {
      float sum = 0.f;
      if (ar) sum += to_f32(ar[c]);
      if (br) sum += to_f32(br[c]);
      if (bias) sum += bias[c];
      value = x[c] + scale * sum;
      if (shift) value += shift[c];
      squares += value * value;
    }
    if (!rows) x[c] = value;
    if (n < KEEP) kept[n] = value;
  }
  if (!weight) return;
  float inv;
  double inv_wide = 0.0;
  if constexpr (WIDE) {
    inv_wide = 1.0 / sqrt(block_sum_wide(squares_wide, scratch_wide) / (double)hidden + (double)eps);
    inv = (float)inv_wide;
  } else {
    inv = rsqrtf(block_sum(squares, scratch) / (float)hidden + eps);
  }
  T* o = out + (int64_t)r * hidden;
  n = 0;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x, ++n) {
    float value;
    if (n < KEEP) {
      value = kept[n];
    } else if (!rows) {
      value = x[c];
    } else {  // recompute: the stream was not written
      if constexpr (WIDE) {
        double sum = 0.0;
        if (ar) sum += (double)ar[c];
        if (br) sum += (double)br[c];
        if (bias) sum += (double)bias[c];
        double v = (double)x[c] + (double)scale * sum;
        if (shift) v += (double)shift[c];
        value = (float)v;
      } else {
        float sum = 0.f;
        if (ar) sum += to_f32(ar[c]);
        if (br) sum += to_f32(br[c]);
        if (bias) sum += bias[c];
        value = x[c] + scale * sum;
        if (shift) value += shift[c];
      }
    }
    if constexpr (WIDE) o[c] = (float)((double)value * inv_wide * (double)weight[c]);
    else o[c] = from_f32<T>(value * inv * to_f32(weight[c]));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void clamped_glu_kernel(const T* __restrict__ gate_up, int64_t in_stride,
                                                          const float* __restrict__ bias, T* __restrict__ out,
                                                          int64_t out_stride, int inter, float limit, float slope) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= inter) return;
  const T* row = gate_up + (int64_t)t * in_stride;
  if constexpr (sizeof(T) == 4) {
    double g = (double)row[c] + (bias ? (double)bias[c] : 0.0);
    double u = (double)row[inter + c] + (bias ? (double)bias[inter + c] : 0.0);
    g = fmin(g, (double)limit);
    u = fmin(fmax(u, -(double)limit), (double)limit);
    out[(int64_t)t * out_stride + c] = (float)(g / (1.0 + exp(-(double)slope * g)) * (u + 1.0));
  } else {
    float g = to_f32(row[c]) + (bias ? bias[c] : 0.f);
    float u = to_f32(row[inter + c]) + (bias ? bias[inter + c] : 0.f);
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    out[(int64_t)t * out_stride + c] = from_f32<T>(g * mi_logistic(slope * g) * (u + 1.f));
  }
}

}  // namespace

// a, b: [rows of the stream, hidden] in the element type with row strides, or null; bias, shift:
// float32 [hidden] or null; weight (element type) with out [num_out_rows, hidden], or both null
// (no norm); rows: int32 [num_out_rows] or null (every row of the stream, num_out_rows of them).
extern "C" int mi_stream_update_norm(int dtype, const void* a, int64_t a_stride, const void* b, int64_t b_stride,
                                     const float* bias, const float* shift, float scale, float* stream,
                                     const void* weight, void* out, const int* rows, int num_out_rows, int hidden,
                                     float eps, hipStream_t stream_handle) {
  MI_REQUIRE(num_out_rows >= 0 && hidden > 0, "stream_update_norm: bad sizes rows=%d hidden=%d", num_out_rows, hidden);
  MI_REQUIRE(stream != nullptr, "stream_update_norm: no stream");
  MI_REQUIRE((weight == nullptr) == (out == nullptr), "stream_update_norm: a norm weight and an output go together");
  MI_REQUIRE(weight != nullptr || rows == nullptr, "stream_update_norm: a row list only makes sense with the norm");
  MI_REQUIRE(weight == nullptr || eps > 0.f, "stream_update_norm: eps must be positive, got %g", (double)eps);
  MI_REQUIRE((!a || a_stride >= hidden) && (!b || b_stride >= hidden), "stream_update_norm: row strides shorter than a row");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "stream_update_norm: unknown dtype %d", dtype);
  if (num_out_rows == 0) return MI_OK;
  const int threads = (num_out_rows <= 64 && hidden >= 2048) ? 1024 : 256;
  if (dtype == MI_F32)
    stream_update_norm_kernel<float><<<num_out_rows, threads, 0, stream_handle>>>(
        (const float*)a, a_stride, (const float*)b, b_stride, bias, shift, scale, stream, (const float*)weight,
        (float*)out, rows, hidden, eps);
  else
    stream_update_norm_kernel<bf16_t><<<num_out_rows, threads, 0, stream_handle>>>(
        (const bf16_t*)a, a_stride, (const bf16_t*)b, b_stride, bias, shift, scale, stream, (const bf16_t*)weight,
        (bf16_t*)out, rows, hidden, eps);
  MI_CHECK_LAUNCH("stream_update_norm");
  return MI_OK;
}

// gate_up [tokens, 2 * inter] (row stride), bias float32 [2 * inter] or null -> out [tokens, inter]
extern "C" int mi_clamped_glu(int dtype, const void* gate_up, int64_t in_stride, const float* bias, void* out,
                              int64_t out_stride, int num_tokens, int inter, float limit, float slope,
                              hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && inter > 0, "clamped_glu: bad sizes tokens=%d inter=%d", num_tokens, inter);
  MI_REQUIRE(in_stride >= 2 * (int64_t)inter && out_stride >= inter, "clamped_glu: row strides shorter than a row");
  MI_REQUIRE(limit > 0.f, "clamped_glu: the limit must be positive, got %g", (double)limit);
  MI_REQUIRE(num_tokens <= 65535 * 64, "clamped_glu: too many tokens");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "clamped_glu: unknown dtype %d", dtype);
  if (num_tokens == 0) return MI_OK;
  // (rows along y in slices of at most 65535)
  for (int first = 0; first < num_tokens; first += 65535) {
    const int count = min(65535, num_tokens - first);
    dim3 grid(ceil_div(inter, 256), count);
    if (dtype == MI_F32)
      clamped_glu_kernel<float><<<grid, 256, 0, stream>>>((const float*)gate_up + (int64_t)first * in_stride, in_stride, bias,
                                                          (float*)out + (int64_t)first * out_stride, out_stride, inter,
                                                          limit, slope);
    else
      clamped_glu_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)gate_up + (int64_t)first * in_stride, in_stride,
                                                           bias, (bf16_t*)out + (int64_t)first * out_stride, out_stride,
                                                           inter, limit, slope);
  }
  MI_CHECK_LAUNCH("clamped_glu");
  return MI_OK;
}
