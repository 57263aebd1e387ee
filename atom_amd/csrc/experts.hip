// A feed-forward of routed experts: every token is sent to `top` of `experts` small gated feed-forwards and
// receives the weighted sum of their outputs.
//
//   router_choose     from float32 router logits z: s = sigmoid(z); the `top` experts with the largest s + correction
//                     are chosen (ties: the lower index); a chosen expert's weight is its s, or s divided by the
//                     chosen experts' sum when `renormalize` is set
//   experts_gate_up   for every (token, choice): act = f(W_gate[e] x) * (W_up[e] x), W stored [experts, 2 ff, width]
//   experts_down      y[t] = sum over the token's choices, in their order, of weight * W_down[e] act
//
// The last two read an expert's rows once per (token, choice): the form for steps of few tokens.  Every sum runs in a
// fixed order over a token's own data, so a token's result does not depend on what else is in the batch.
#include "common.h"

__global__ void router_choose_kernel(const float* __restrict__ logits, const float* __restrict__ correction,
                                     int* __restrict__ ids, float* __restrict__ weights, int tokens, int experts,
                                     int top, int renormalize) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= tokens) return;
  const float* z = logits + (size_t)t * experts;
  int* mine = ids + (size_t)t * top;
  float* w = weights + (size_t)t * top;
  float total = 0.f;
  for (int k = 0; k < top; ++k) {
    int best = -1;
    float best_score = -INFINITY, best_s = 0.f;
    for (int e = 0; e < experts; ++e) {
      bool taken = false;
      for (int j = 0; j < k; ++j) taken |= (mine[j] == e);
      if (taken) continue;
      const float s = 1.f / (1.f + expf(-z[e]));
      const float score = s + (correction ? correction[e] : 0.f);
      if (best < 0 || score > best_score) {
        best = e;
        best_score = score;
        best_s = s;
      }
    }
    mine[k] = best;
    w[k] = best_s;
    total += best_s;
  }
  if (renormalize)
    for (int k = 0; k < top; ++k) w[k] /= total;
}

ATOM_EXPORT int atom_router_choose(const float* logits, const float* correction, int* ids, float* weights, int tokens,
                                   int experts, int top, int renormalize, hipStream_t stream) {
  if (tokens < 0 || experts <= 0 || top <= 0 || top > experts) return ATOM_BAD_SHAPE;
  if (logits == nullptr || ids == nullptr || weights == nullptr) return ATOM_BAD_SHAPE;
  if (tokens == 0) return ATOM_OK;
  hipLaunchKernelGGL(router_choose_kernel, dim3((tokens + 127) / 128), dim3(128), 0, stream, logits, correction, ids,
                     weights, tokens, experts, top, renormalize);
  return launch_status();
}

__device__ __forceinline__ float expert_activation(float g, int act) {
  if (act == 1) return g > 0.f ? g : 0.f;
  if (act == 2) return 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
  return g / (1.f + expf(-g));
}

constexpr int kExpCols = 32;   // output columns of a block: 4 waves x 8

template <typename T, typename TW>
__global__ void __launch_bounds__(256)
experts_gate_up_kernel(const T* __restrict__ x, const TW* __restrict__ w, const int* __restrict__ ids,
                       T* __restrict__ act_out, int top, int ff, int width, int act) {
  extern __shared__ float xs[];   // width
  const int pair = blockIdx.x;
  const int t = pair / top;
  const int e = ids[pair];
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const T* xr = x + (size_t)t * width;
  for (int i = tid; i < width; i += 256) xs[i] = to_f32(xr[i]);
  __syncthreads();
  const TW* we = w + (size_t)e * 2 * ff * width;
  for (int c = 0; c < kExpCols / 4; ++c) {
    const int col = blockIdx.y * kExpCols + wave * (kExpCols / 4) + c;
    if (col >= ff) break;
    const TW* gr = we + (size_t)col * width;
    const TW* ur = we + (size_t)(ff + col) * width;
    float g = 0.f, u = 0.f;
    for (int i = lane; i < width; i += kWave) {
      const float xv = xs[i];
      g = fmaf(xv, to_f32(gr[i]), g);
      u = fmaf(xv, to_f32(ur[i]), u);
    }
    g = wave_sum(g);
    u = wave_sum(u);
    if (lane == 0) act_out[(size_t)pair * ff + col] = from_f32<T>(expert_activation(g, act) * u);
  }
}

template <typename T, typename TW>
__global__ void __launch_bounds__(256)
experts_down_kernel(const T* __restrict__ act_in, const TW* __restrict__ w, const int* __restrict__ ids,
                    const float* __restrict__ weights, T* __restrict__ y, int top, int ff, int width) {
  extern __shared__ float as[];   // top * ff
  const int t = blockIdx.x;
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  for (int i = tid; i < top * ff; i += 256) as[i] = to_f32(act_in[(size_t)t * top * ff + i]);
  __syncthreads();
  for (int c = 0; c < kExpCols / 4; ++c) {
    const int col = blockIdx.y * kExpCols + wave * (kExpCols / 4) + c;
    if (col >= width) break;
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
      const int e = ids[(size_t)t * top + k];
      const TW* wr = w + ((size_t)e * width + col) * ff;
      float s = 0.f;
      for (int i = lane; i < ff; i += kWave) s = fmaf(as[k * ff + i], to_f32(wr[i]), s);
      total += weights[(size_t)t * top + k] * wave_sum(s);
    }
    if (lane == 0) y[(size_t)t * width + col] = from_f32<T>(total);
  }
}

ATOM_EXPORT int atom_experts_gate_up(const void* x, const void* w, int w_dtype, const int* ids, void* act_out, int dtype,
                                     int tokens, int top, int ff, int width, int act, hipStream_t stream) {
  if (tokens < 0 || top <= 0 || ff <= 0 || width <= 0 || act < 0 || act > 2) return ATOM_BAD_SHAPE;
  if (x == nullptr || w == nullptr || ids == nullptr || act_out == nullptr) return ATOM_BAD_SHAPE;
  if ((size_t)width * sizeof(float) > 64 * 1024) return ATOM_TOO_LARGE;
  if (tokens == 0) return ATOM_OK;
  dim3 grid(tokens * top, (ff + kExpCols - 1) / kExpCols), block(256);
  if (grid.y > 65535) return ATOM_TOO_LARGE;
  const size_t smem = (size_t)width * sizeof(float);
#define LAUNCH(T, TW)                                                                                              \
  hipLaunchKernelGGL((experts_gate_up_kernel<T, TW>), grid, block, smem, stream, (const T*)x, (const TW*)w, ids, \
                     (T*)act_out, top, ff, width, act)
  if (dtype == ATOM_F32 && w_dtype == ATOM_F32) LAUNCH(float, float);
  else if (dtype == ATOM_BF16 && w_dtype == ATOM_BF16) LAUNCH(bf16_t, bf16_t);
  else if (dtype == ATOM_BF16 && w_dtype == ATOM_F32) LAUNCH(bf16_t, float);
  else return ATOM_BAD_DTYPE;
#undef LAUNCH
  return launch_status();
}

ATOM_EXPORT int atom_experts_down(const void* act_in, const void* w, int w_dtype, const int* ids, const float* weights,
                                  void* y, int dtype, int tokens, int top, int ff, int width, hipStream_t stream) {
  if (tokens < 0 || top <= 0 || ff <= 0 || width <= 0) return ATOM_BAD_SHAPE;
  if (act_in == nullptr || w == nullptr || ids == nullptr || weights == nullptr || y == nullptr) return ATOM_BAD_SHAPE;
  if ((size_t)top * ff * sizeof(float) > 64 * 1024) return ATOM_TOO_LARGE;
  if (tokens == 0) return ATOM_OK;
  dim3 grid(tokens, (width + kExpCols - 1) / kExpCols), block(256);
  if (grid.y > 65535) return ATOM_TOO_LARGE;
  const size_t smem = (size_t)top * ff * sizeof(float);
#define LAUNCH(T, TW)                                                                                               \
  hipLaunchKernelGGL((experts_down_kernel<T, TW>), grid, block, smem, stream, (const T*)act_in, (const TW*)w, ids, \
                     weights, (T*)y, top, ff, width)
  if (dtype == ATOM_F32 && w_dtype == ATOM_F32) LAUNCH(float, float);
  else if (dtype == ATOM_BF16 && w_dtype == ATOM_BF16) LAUNCH(bf16_t, bf16_t);
  else if (dtype == ATOM_BF16 && w_dtype == ATOM_F32) LAUNCH(bf16_t, float);
  else return ATOM_BAD_DTYPE;
#undef LAUNCH
  return launch_status();
}
