// Layer norm with weight and bias, and the small kernels that feed or leave the float32 residual stream.
//
//   y = (x - mean(x)) / sqrt(mean((x - mean(x))^2) + eps) * w + b          all in float32
//
// One block per row; the row sits in LDS as float32 between the passes (mean, then the mean of the
// squared deviations, then the output), so the variance is the two-pass one.
//
// modes of atom_layernorm:
//   0 plain  y = LN(x)
//   1 init   residual = x;  y = LN(x)
//   2 add    residual += x; y = LN(residual)
//   3 post   residual += LN(x; w, b); y = LN(residual; w2, b2)     (y may be null: the sum alone)
// With `rows` (modes 0 and 2) only those source rows are normed, into y[0 .. n), and the residual is
// not written.  The input and the output have element types of their own.
#include "common.h"

constexpr int kNormThreads = 256;

template <typename TX, typename TY>
__global__ void __launch_bounds__(kNormThreads)
layernorm_kernel(const TX* __restrict__ x, float* __restrict__ residual, const float* __restrict__ w,
                 const float* __restrict__ b, const float* __restrict__ w2, const float* __restrict__ b2,
                 TY* __restrict__ y, const int* __restrict__ rows, int width, float eps, int mode) {
  extern __shared__ float smem[];
  float* row = smem;            // width
  float* scratch = smem + width;  // 16
  const int tid = threadIdx.x;
  const size_t src = rows ? (size_t)rows[blockIdx.x] : (size_t)blockIdx.x;
  const size_t dst = blockIdx.x;
  const TX* xr = x + src * width;
  float* rr = residual ? residual + src * width : nullptr;
  const float inv_width = 1.f / (float)width;

  float part = 0.f;
  for (int i = tid; i < width; i += kNormThreads) {
    float v = to_f32(xr[i]);
    if (mode == 2) v += rr[i];
    row[i] = v;
    part += v;
  }
  if (mode == 1 || (mode == 2 && rows == nullptr)) {
    for (int i = tid; i < width; i += kNormThreads) rr[i] = row[i];
  }
  float mean = block_sum(part, scratch) * inv_width;
  part = 0.f;
  for (int i = tid; i < width; i += kNormThreads) {
    const float dlt = row[i] - mean;
    part += dlt * dlt;
  }
  float rstd = 1.f / sqrtf(block_sum(part, scratch) * inv_width + eps);
  if (mode != 3) {
    TY* yr = y + dst * width;
    for (int i = tid; i < width; i += kNormThreads) yr[i] = from_f32<TY>((row[i] - mean) * rstd * w[i] + b[i]);
    return;
  }
  // post: the normed row joins the stream, and the stream is normed for what follows
  part = 0.f;
  for (int i = tid; i < width; i += kNormThreads) {
    const float v = rr[i] + ((row[i] - mean) * rstd * w[i] + b[i]);
    rr[i] = v;
    row[i] = v;
    part += v;
  }
  if (y == nullptr) return;
  mean = block_sum(part, scratch) * inv_width;
  part = 0.f;
  for (int i = tid; i < width; i += kNormThreads) {
    const float dlt = row[i] - mean;
    part += dlt * dlt;
  }
  rstd = 1.f / sqrtf(block_sum(part, scratch) * inv_width + eps);
  TY* yr = y + dst * width;
  for (int i = tid; i < width; i += kNormThreads) yr[i] = from_f32<TY>((row[i] - mean) * rstd * w2[i] + b2[i]);
}

ATOM_EXPORT int atom_layernorm(const void* x, int x_dtype, float* residual, const float* w, const float* b,
                               const float* w2, const float* b2, void* y, int y_dtype, const int* rows, int num_rows,
                               int width, float eps, int mode, hipStream_t stream) {
  if (num_rows < 0 || width <= 0 || mode < 0 || mode > 3) return ATOM_BAD_SHAPE;
  if (x == nullptr || w == nullptr || b == nullptr) return ATOM_BAD_SHAPE;
  if (mode != 0 && residual == nullptr) return ATOM_BAD_SHAPE;
  if (mode != 3 && y == nullptr) return ATOM_BAD_SHAPE;
  if (mode == 3 && y != nullptr && (w2 == nullptr || b2 == nullptr)) return ATOM_BAD_SHAPE;
  if (rows != nullptr && (mode == 1 || mode == 3)) return ATOM_BAD_SHAPE;
  if ((unsigned)x_dtype > 1u || (unsigned)y_dtype > 1u) return ATOM_BAD_DTYPE;
  if ((size_t)(width + 16) * sizeof(float) > 160 * 1024) return ATOM_TOO_LARGE;
  if (num_rows == 0) return ATOM_OK;
  const size_t smem = (size_t)(width + 16) * sizeof(float);
  dim3 grid(num_rows), block(kNormThreads);
#define LAUNCH(TX, TY)                                                                                       \
  hipLaunchKernelGGL((layernorm_kernel<TX, TY>), grid, block, smem, stream, (const TX*)x, residual, w, b, w2, b2, \
                     (TY*)y, rows, width, eps, mode)
  switch (x_dtype * 2 + y_dtype) {
    case 0: LAUNCH(float, float); break;
    case 1: LAUNCH(float, bf16_t); break;
    case 2: LAUNCH(bf16_t, float); break;
    default: LAUNCH(bf16_t, bf16_t); break;
  }
#undef LAUNCH
  return launch_status();
}

// ------------------------------------------------------------------ embedding rows times a constant, float32 out

template <typename TT>
__global__ void embedding_scaled_kernel(const TT* __restrict__ table, const int* __restrict__ ids,
                                        float* __restrict__ out, int hidden, int vocab, float scale) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const TT* src = table + (size_t)id * hidden;
  float* dst = out + (size_t)t * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_f32(src[i]) * scale;
}

ATOM_EXPORT int atom_embedding_scaled(const void* table, int table_dtype, const int* ids, float* out, int tokens,
                                      int hidden, int vocab, float scale, hipStream_t stream) {
  if (tokens < 0 || hidden <= 0 || vocab <= 0) return ATOM_BAD_SHAPE;
  if (tokens == 0) return ATOM_OK;
  ATOM_DISPATCH_DTYPE(table_dtype, hipLaunchKernelGGL((embedding_scaled_kernel<T>), dim3(tokens), dim3(256), 0, stream,
                                                       (const T*)table, ids, out, hidden, vocab, scale));
  return launch_status();
}

// ------------------------------------------------------------------ [stream ; first] side by side
//
// out[t] = [ residual[t] + hidden[t] ; first[t] ]: the residual stream (its pending summand added) beside another
// float32 row, as the input of one product.  `residual` may be null (hidden alone).

template <typename TH, typename TO>
__global__ void sum_concat_kernel(const TH* __restrict__ hidden, const float* __restrict__ residual,
                                  const float* __restrict__ first, TO* __restrict__ out, int width) {
  const size_t t = blockIdx.x;
  const TH* h = hidden + t * width;
  const float* f = first + t * width;
  TO* o = out + t * 2 * (size_t)width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = to_f32(h[i]);
    if (residual) v += residual[t * width + i];
    o[i] = from_f32<TO>(v);
    o[width + i] = from_f32<TO>(f[i]);
  }
}

ATOM_EXPORT int atom_sum_concat(const void* hidden, int hidden_dtype, const float* residual, const float* first,
                                void* out, int out_dtype, int tokens, int width, hipStream_t stream) {
  if (tokens < 0 || width <= 0 || hidden == nullptr || first == nullptr || out == nullptr) return ATOM_BAD_SHAPE;
  if ((unsigned)hidden_dtype > 1u || (unsigned)out_dtype > 1u) return ATOM_BAD_DTYPE;
  if (tokens == 0) return ATOM_OK;
  dim3 grid(tokens), block(256);
#define LAUNCH(TH, TO) \
  hipLaunchKernelGGL((sum_concat_kernel<TH, TO>), grid, block, 0, stream, (const TH*)hidden, residual, first, (TO*)out, width)
  switch (hidden_dtype * 2 + out_dtype) {
    case 0: LAUNCH(float, float); break;
    case 1: LAUNCH(float, bf16_t); break;
    case 2: LAUNCH(bf16_t, float); break;
    default: LAUNCH(bf16_t, bf16_t); break;
  }
#undef LAUNCH
  return launch_status();
}

// ------------------------------------------------------------------ act(gate) * up for activations other than SiLU
//
// x [rows, 2 * inter] = gate | up.  act: 0 SiLU, 1 ReLU, 2 GELU (tanh form).

__device__ __forceinline__ float gate_activation(float g, int act) {
  if (act == 1) return g > 0.f ? g : 0.f;
  if (act == 2) return 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
  return g / (1.f + expf(-g));
}

template <typename T>
__global__ void gated_act_kernel(const T* __restrict__ x, T* __restrict__ y, int inter, size_t total, int act) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t row = idx / inter;
  const int col = (int)(idx - row * inter);
  const float g = to_f32(x[row * 2 * inter + col]);
  const float u = to_f32(x[row * 2 * inter + inter + col]);
  y[idx] = from_f32<T>(gate_activation(g, act) * u);
}

ATOM_EXPORT int atom_gated_act(const void* x, void* y, int dtype, int rows, int inter, int act, hipStream_t stream) {
  if (rows < 0 || inter <= 0 || act < 0 || act > 2 || x == nullptr || y == nullptr) return ATOM_BAD_SHAPE;
  const size_t total = (size_t)rows * inter;
  if (total == 0) return ATOM_OK;
  const size_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffu) return ATOM_TOO_LARGE;
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((gated_act_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream,
                                                 (const T*)x, (T*)y, inter, total, act));
  return launch_status();
}
