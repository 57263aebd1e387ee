// The real-gated linear recurrence, token by token and channel by channel, in float32:
//
//   r = sigmoid(gr + br);  i = sigmoid(gi + bi);  log a = -scale * r * softplus(lam);  a = exp(log a)
//   S <- a S + sqrt(1 - a^2) (i u);   out = S * gelu_tanh(y)
//
// gr and gi are the gates' small products (before their biases), u the convolved input branch, y the other branch
// before its activation.  S [channels] sits in a request's state row at state_off and starts from what the slot
// holds (zero for a new request).  1 - a^2 is formed as -expm1(2 log a), which keeps its digits when a is near 1.
//
// Requests are walked through the step's device arrays, so prompt portions, single tokens and padded rows
// (slot < 0: nothing of the state is touched, zeros are written) run the same kernel.  A thread owns a channel of a
// request; the loads of the tokens ahead do not depend on S, so they are in flight while the chain runs.
#include "common.h"

__device__ __forceinline__ float gelu_tanh_y(float z) {
  const float inner = 0.7978845608028654f * (z + 0.044715f * z * z * z);
  return 0.5f * z * (1.f + tanhf(inner));
}

template <typename TO>
__global__ void __launch_bounds__(128)
rglru_scan_kernel(const float* __restrict__ u, const float* __restrict__ gr, const float* __restrict__ gi,
                  const float* __restrict__ br, const float* __restrict__ bi, const float* __restrict__ lam,
                  const float* __restrict__ y, int ld_y, int y_off, float* __restrict__ state, long slot_stride,
                  long state_off, const int* __restrict__ cu_seqlens, const int* __restrict__ slot_of_seq,
                  TO* __restrict__ out, int channels, float scale) {
  const int c = blockIdx.x * 128 + threadIdx.x;
  const int seq = blockIdx.y;
  if (c >= channels) return;
  const int begin = cu_seqlens[seq], end = cu_seqlens[seq + 1];
  const int slot = slot_of_seq[seq];
  if (slot < 0) {
    for (int t = begin; t < end; ++t) out[(size_t)t * channels + c] = from_f32<TO>(0.f);
    return;
  }
  float* sp = state + (size_t)slot * slot_stride + state_off + c;
  float S = *sp;
  const float l = lam[c];
  const float rate = -scale * (l > 20.f ? l : log1pf(expf(l)));
  const float rb = br[c], ib = bi[c];
#pragma unroll 4
  for (int t = begin; t < end; ++t) {
    const size_t at = (size_t)t * channels + c;
    const float r = 1.f / (1.f + expf(-(gr[at] + rb)));
    const float g = 1.f / (1.f + expf(-(gi[at] + ib)));
    const float log_a = rate * r;
    const float a = expf(log_a);
    const float mult = sqrtf(-expm1f(2.f * log_a));
    S = fmaf(a, S, mult * (g * u[at]));
    out[at] = from_f32<TO>(S * gelu_tanh_y(y[(size_t)t * ld_y + y_off + c]));
  }
  *sp = S;
}

ATOM_EXPORT int atom_rglru_scan(const float* u, const float* gr, const float* gi, const float* br, const float* bi,
                                const float* lam, const float* y, int ld_y, int y_off, float* state, long slot_stride,
                                long state_off, const int* cu_seqlens, const int* slot_of_seq, int num_seqs, void* out,
                                int out_dtype, int channels, float scale, hipStream_t stream) {
  if (channels <= 0 || num_seqs < 0 || y_off < 0 || y_off + channels > ld_y) return ATOM_BAD_SHAPE;
  if (state_off < 0 || slot_stride < state_off + channels) return ATOM_BAD_SHAPE;
  if (u == nullptr || gr == nullptr || gi == nullptr || br == nullptr || bi == nullptr || lam == nullptr ||
      y == nullptr || state == nullptr || cu_seqlens == nullptr || slot_of_seq == nullptr || out == nullptr)
    return ATOM_BAD_SHAPE;
  if (num_seqs == 0) return ATOM_OK;
  if (num_seqs > 65535) return ATOM_TOO_LARGE;
  dim3 grid((channels + 127) / 128, num_seqs), block(128);
  ATOM_DISPATCH_DTYPE(out_dtype, hipLaunchKernelGGL((rglru_scan_kernel<T>), grid, block, 0, stream, u, gr, gi, br, bi,
                                                     lam, y, ld_y, y_off, state, slot_stride, state_off, cu_seqlens,
                                                     slot_of_seq, (T*)out, channels, scale));
  return launch_status();
}
