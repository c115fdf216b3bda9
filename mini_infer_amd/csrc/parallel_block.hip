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

typedef bf16_t bf16x4_t __attribute__((ext_vector_type(4)));

// VEC consecutive elements at once (VEC = 4: 16-byte float32 and 8-byte bfloat16 accesses)
template <int VEC>
__device__ __forceinline__ void load_some(const float* p, float v[VEC]) {
  if constexpr (VEC == 4) {
    const float4 x = *reinterpret_cast<const float4*>(p);
    v[0] = x.x, v[1] = x.y, v[2] = x.z, v[3] = x.w;
  } else {
    v[0] = p[0];
  }
}
template <int VEC>
__device__ __forceinline__ void load_some(const bf16_t* p, float v[VEC]) {
  if constexpr (VEC == 4) {
    const bf16x4_t x = *reinterpret_cast<const bf16x4_t*>(p);
    v[0] = (float)x[0], v[1] = (float)x[1], v[2] = (float)x[2], v[3] = (float)x[3];
  } else {
    v[0] = (float)p[0];
  }
}
template <int VEC>
__device__ __forceinline__ void store_some(float* p, const float v[VEC]) {
  if constexpr (VEC == 4) *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  else p[0] = v[0];
}
template <int VEC>
__device__ __forceinline__ void store_some(bf16_t* p, const float v[VEC]) {
  if constexpr (VEC == 4) {
    bf16x4_t x;
    x[0] = (bf16_t)v[0], x[1] = (bf16_t)v[1], x[2] = (bf16_t)v[2], x[3] = (bf16_t)v[3];
    *reinterpret_cast<bf16x4_t*>(p) = x;
  } else {
    p[0] = (bf16_t)v[0];
  }
}

// The new values of VEC columns of a row: x + scale * (a + b + bias) + shift.
template <typename T, int VEC>
__device__ __forceinline__ void updated(const T* ar, const T* br, const float* bias, const float* shift, float scale,
                                        const float* x, int c, float value[VEC]) {
  float xv[VEC], av[VEC], bv[VEC], cv[VEC], sv[VEC];
  load_some<VEC>(x + c, xv);
#pragma unroll
  for (int e = 0; e < VEC; ++e) av[e] = bv[e] = cv[e] = sv[e] = 0.f;
  if (ar) load_some<VEC>(ar + c, av);
  if (br) load_some<VEC>(br + c, bv);
  if (bias) load_some<VEC>(bias + c, cv);
  if (shift) load_some<VEC>(shift + c, sv);
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    if constexpr (sizeof(T) == 4) value[e] = (float)((double)xv[e] + (double)scale * (((double)av[e] + (double)bv[e]) + (double)cv[e]) + (double)sv[e]);
    else value[e] = xv[e] + scale * ((av[e] + bv[e]) + cv[e]) + sv[e];
  }
}

// One block a row.  `rows` (optional) lists the rows to norm; with it the stream is left as
// it was (the rows' new values are used for the norm only), as the final norm wants it.
template <typename T, int VEC>
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
  // a thread keeps the new values of its first columns (wider rows are made again below)
  constexpr int KEEP = 4;
  float kept[KEEP][VEC];
  float squares = 0.f;
  double squares_wide = 0.0;
  int n = 0;
  for (int c = threadIdx.x * VEC; c < hidden; c += blockDim.x * VEC, ++n) {
    float value[VEC];
    updated<T, VEC>(ar, br, bias, shift, scale, x, c, value);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      if constexpr (WIDE) squares_wide += (double)value[e] * (double)value[e];
      else squares += value[e] * value[e];
    }
    if (!rows) store_some<VEC>(x + c, value);
    if (n < KEEP) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) kept[n][e] = value[e];
    }
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
  for (int c = threadIdx.x * VEC; c < hidden; c += blockDim.x * VEC, ++n) {
    float value[VEC], w[VEC];
    if (n < KEEP) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) value[e] = kept[n][e];
    } else if (!rows) {
      load_some<VEC>(x + c, value);
    } else {  // made again: the stream was not written
      updated<T, VEC>(ar, br, bias, shift, scale, x, c, value);
    }
    load_some<VEC>(weight + c, w);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      if constexpr (WIDE) value[e] = (float)((double)value[e] * inv_wide * (double)w[e]);
      else value[e] = value[e] * inv * w[e];
    }
    store_some<VEC>(o + c, value);
  }
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void clamped_glu_kernel(const T* __restrict__ gate_up, int64_t in_stride,
                                                          const float* __restrict__ bias, T* __restrict__ out,
                                                          int64_t out_stride, int inter, float limit, float slope) {
  const int t = blockIdx.y;
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * VEC;
  if (c >= inter) return;
  const T* row = gate_up + (int64_t)t * in_stride;
  float g[VEC], u[VEC], bg[VEC], bu[VEC], y[VEC];
  load_some<VEC>(row + c, g);
  load_some<VEC>(row + inter + c, u);
#pragma unroll
  for (int e = 0; e < VEC; ++e) bg[e] = bu[e] = 0.f;
  if (bias) {
    load_some<VEC>(bias + c, bg);
    load_some<VEC>(bias + inter + c, bu);
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    if constexpr (sizeof(T) == 4) {
      double gd = fmin((double)g[e] + (double)bg[e], (double)limit);
      double ud = fmin(fmax((double)u[e] + (double)bu[e], -(double)limit), (double)limit);
      y[e] = (float)(gd / (1.0 + exp(-(double)slope * gd)) * (ud + 1.0));
    } else {
      const float gf = fminf(g[e] + bg[e], limit);
      const float uf = fminf(fmaxf(u[e] + bu[e], -limit), limit);
      y[e] = gf * mi_logistic(slope * gf) * (uf + 1.f);
    }
  }
  store_some<VEC>(out + (int64_t)t * out_stride + c, y);
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
  // four columns a thread where every row begins on a 16-byte boundary
  const size_t elem = dtype == MI_F32 ? 4 : 2;
  const bool vec = hidden % 4 == 0 && ((uintptr_t)a | (uintptr_t)b | (uintptr_t)weight | (uintptr_t)out | (uintptr_t)(a_stride * elem) |
                                       (uintptr_t)(b_stride * elem)) % 16 == 0 &&
                   ((uintptr_t)bias | (uintptr_t)shift | (uintptr_t)stream) % 16 == 0;
#define MI_UPDATE_LAUNCH(T, VEC)                                                                                      \
  stream_update_norm_kernel<T, VEC><<<num_out_rows, threads, 0, stream_handle>>>(                                     \
      (const T*)a, a_stride, (const T*)b, b_stride, bias, shift, scale, stream, (const T*)weight, (T*)out, rows, hidden, eps)
  if (dtype == MI_F32) { if (vec) MI_UPDATE_LAUNCH(float, 4); else MI_UPDATE_LAUNCH(float, 1); }
  else { if (vec) MI_UPDATE_LAUNCH(bf16_t, 4); else MI_UPDATE_LAUNCH(bf16_t, 1); }
#undef MI_UPDATE_LAUNCH
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
  const size_t elem = dtype == MI_F32 ? 4 : 2;
  const bool vec = inter % 4 == 0 && ((uintptr_t)gate_up | (uintptr_t)out | (uintptr_t)(in_stride * elem) | (uintptr_t)(out_stride * elem) |
                                      (uintptr_t)(inter * elem)) % 16 == 0 && (uintptr_t)bias % 16 == 0;
  // (rows along y in slices of at most 65535)
  for (int first = 0; first < num_tokens; first += 65535) {
    const int count = min(65535, num_tokens - first);
    dim3 grid(ceil_div(inter, 256 * (vec ? 4 : 1)), count);
#define MI_GLU_LAUNCH(T, VEC)                                                                                          \
  clamped_glu_kernel<T, VEC><<<grid, 256, 0, stream>>>((const T*)gate_up + (int64_t)first * in_stride, in_stride, bias, \
                                                       (T*)out + (int64_t)first * out_stride, out_stride, inter, limit, slope)
    if (dtype == MI_F32) { if (vec) MI_GLU_LAUNCH(float, 4); else MI_GLU_LAUNCH(float, 1); }
    else { if (vec) MI_GLU_LAUNCH(bf16_t, 4); else MI_GLU_LAUNCH(bf16_t, 1); }
#undef MI_GLU_LAUNCH
  }
  MI_CHECK_LAUNCH("clamped_glu");
  return MI_OK;
}
