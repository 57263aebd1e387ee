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
// (slot < 0: nothing of the state is touched, zeros are written) run the same kernels.
//
// Short requests (up to 64 tokens each): one kernel, a thread owns a channel of a request and walks its tokens; the
// loads of the tokens ahead do not depend on S, so they are in flight while the chain runs.
// Longer ones: the recurrence is linear in S, so a run of 64 tokens acts on it as S -> A S + B with A the product
// of the run's decays and B what the run leaves of a zero state.  A first kernel forms (A, B) of every run (and
// copies the state S had before the step aside), a second one starts every run from the state before the step
// folded through the runs ahead of it, and walks the run's tokens.  Both have a block per (128 channels, request,
// run), so a prompt fills the chip instead of one wave per 64 channels walking all of it.
#include "common.h"

__device__ __forceinline__ float gelu_tanh_y(float z) {
  const float inner = 0.7978845608028654f * (z + 0.044715f * z * z * z);
  return 0.5f * z * (1.f + tanhf(inner));
}

struct Step {
  float a, b;
};

// One token's decay and input: S <- a S + b.
__device__ __forceinline__ Step token_step(float gr, float gi, float u, float rb, float ib, float rate) {
  const float r = 1.f / (1.f + expf(-(gr + rb)));
  const float g = 1.f / (1.f + expf(-(gi + ib)));
  const float log_a = rate * r;
  Step s;
  s.a = expf(log_a);
  s.b = sqrtf(-expm1f(2.f * log_a)) * (g * u);
  return s;
}

constexpr int kScanRun = 64;

// grid (channel blocks, requests, runs).  ab [requests, runs, 2, channels]; s0 [requests, channels].
__global__ void __launch_bounds__(128)
rglru_runs_kernel(const float* __restrict__ u, const float* __restrict__ gr, const float* __restrict__ gi,
                  const float* __restrict__ br, const float* __restrict__ bi, const float* __restrict__ lam,
                  const float* __restrict__ state, long slot_stride, long state_off, const int* __restrict__ cu_seqlens,
                  const int* __restrict__ slot_of_seq, float* __restrict__ ab, float* __restrict__ s0, int channels,
                  float scale) {
  const int c = blockIdx.x * 128 + threadIdx.x;
  const int seq = blockIdx.y, run = blockIdx.z, runs = gridDim.z;
  if (c >= channels) return;
  const int slot = slot_of_seq[seq];
  if (slot < 0) return;
  if (run == 0) s0[(size_t)seq * channels + c] = state[(size_t)slot * slot_stride + state_off + c];
  const int begin = cu_seqlens[seq], end = cu_seqlens[seq + 1];
  const int first = begin + run * kScanRun;
  if (first >= end) return;
  const int last = first + kScanRun < end ? first + kScanRun : end;
  const float l = lam[c];
  const float rate = -scale * (l > 20.f ? l : log1pf(expf(l)));
  const float rb = br[c], ib = bi[c];
  float A = 1.f, B = 0.f;
#pragma unroll 4
  for (int t = first; t < last; ++t) {
    const size_t at = (size_t)t * channels + c;
    const Step s = token_step(gr[at], gi[at], u[at], rb, ib, rate);
    A *= s.a;
    B = fmaf(s.a, B, s.b);
  }
  float* dst = ab + ((size_t)seq * runs + run) * 2 * channels + c;
  dst[0] = A;
  dst[channels] = B;
}

template <typename TO>
__global__ void __launch_bounds__(128)
rglru_scan_runs_kernel(const float* __restrict__ u, const float* __restrict__ gr, const float* __restrict__ gi,
                       const float* __restrict__ br, const float* __restrict__ bi, const float* __restrict__ lam,
                       const float* __restrict__ y, int ld_y, int y_off, float* __restrict__ state, long slot_stride,
                       long state_off, const int* __restrict__ cu_seqlens, const int* __restrict__ slot_of_seq,
                       const float* __restrict__ ab, const float* __restrict__ s0, TO* __restrict__ out, int channels,
                       float scale) {
  const int c = blockIdx.x * 128 + threadIdx.x;
  const int seq = blockIdx.y, run = blockIdx.z, runs = gridDim.z;
  if (c >= channels) return;
  const int begin = cu_seqlens[seq], end = cu_seqlens[seq + 1];
  const int first = begin + run * kScanRun;
  if (first >= end) return;
  const int last = first + kScanRun < end ? first + kScanRun : end;
  const int slot = slot_of_seq[seq];
  if (slot < 0) {
    for (int t = first; t < last; ++t) out[(size_t)t * channels + c] = from_f32<TO>(0.f);
    return;
  }
  float S = s0[(size_t)seq * channels + c];
  const float* src = ab + (size_t)seq * runs * 2 * channels + c;
  for (int j = 0; j < run; ++j) S = fmaf(src[(size_t)j * 2 * channels], S, src[(size_t)j * 2 * channels + channels]);
  const float l = lam[c];
  const float rate = -scale * (l > 20.f ? l : log1pf(expf(l)));
  const float rb = br[c], ib = bi[c];
#pragma unroll 4
  for (int t = first; t < last; ++t) {
    const size_t at = (size_t)t * channels + c;
    const Step s = token_step(gr[at], gi[at], u[at], rb, ib, rate);
    S = fmaf(s.a, S, s.b);
    out[at] = from_f32<TO>(S * gelu_tanh_y(y[(size_t)t * ld_y + y_off + c]));
  }
  if (last == end) state[(size_t)slot * slot_stride + state_off + c] = S;
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
    const Step s = token_step(gr[at], gi[at], u[at], rb, ib, rate);
    S = fmaf(s.a, S, s.b);
    out[at] = from_f32<TO>(S * gelu_tanh_y(y[(size_t)t * ld_y + y_off + c]));
  }
  *sp = S;
}

ATOM_EXPORT int atom_rglru_scan(const float* u, const float* gr, const float* gi, const float* br, const float* bi,
                                const float* lam, const float* y, int ld_y, int y_off, float* state, long slot_stride,
                                long state_off, const int* cu_seqlens, const int* slot_of_seq, int num_seqs, void* out,
                                int out_dtype, int channels, float scale, int max_q_len, float* workspace,
                                long workspace_floats, hipStream_t stream) {
  if (channels <= 0 || num_seqs < 0 || y_off < 0 || y_off + channels > ld_y) return ATOM_BAD_SHAPE;
  if (state_off < 0 || slot_stride < state_off + channels) return ATOM_BAD_SHAPE;
  if (u == nullptr || gr == nullptr || gi == nullptr || br == nullptr || bi == nullptr || lam == nullptr ||
      y == nullptr || state == nullptr || cu_seqlens == nullptr || slot_of_seq == nullptr || out == nullptr)
    return ATOM_BAD_SHAPE;
  if (num_seqs == 0) return ATOM_OK;
  if (num_seqs > 65535 || max_q_len < 0) return ATOM_TOO_LARGE;
  if (max_q_len > kScanRun && workspace != nullptr) {
    // runs of 64 tokens side by side; the workspace holds the states before the step, then every run's (A, B)
    const int runs = (max_q_len + kScanRun - 1) / kScanRun;
    if (runs > 65535) return ATOM_TOO_LARGE;
    if (workspace_floats < (long)num_seqs * channels * (1 + 2 * (long)runs)) return ATOM_BAD_SHAPE;
    float* s0 = workspace;
    float* ab = workspace + (size_t)num_seqs * channels;
    dim3 grid((channels + 127) / 128, num_seqs, runs), block(128);
    hipLaunchKernelGGL(rglru_runs_kernel, grid, block, 0, stream, u, gr, gi, br, bi, lam, state, slot_stride, state_off,
                       cu_seqlens, slot_of_seq, ab, s0, channels, scale);
    ATOM_DISPATCH_DTYPE(out_dtype, hipLaunchKernelGGL((rglru_scan_runs_kernel<T>), grid, block, 0, stream, u, gr, gi, br,
                                                       bi, lam, y, ld_y, y_off, state, slot_stride, state_off, cu_seqlens,
                                                       slot_of_seq, ab, s0, (T*)out, channels, scale));
    return launch_status();
  }
  dim3 grid((channels + 127) / 128, num_seqs), block(128);
  ATOM_DISPATCH_DTYPE(out_dtype, hipLaunchKernelGGL((rglru_scan_kernel<T>), grid, block, 0, stream, u, gr, gi, br, bi,
                                                     lam, y, ld_y, y_off, state, slot_stride, state_off, cu_seqlens,
                                                     slot_of_seq, (T*)out, channels, scale));
  return launch_status();
}
