// Attention whose values are its keys: from the float32 product [q | k | ...] of a token,
//
//   q and k are RMS-normed over their whole rows (all heads at once, a weight per entry; no weight: no norm),
//   entries (2i, 2i + 1) of the first rot_dims entries of every head are turned by position * freq[i]
//   (freq float64; the angle is formed in float64 and reduced before its float32 sine and cosine),
//   q goes to q_out [T, H, D]; the normed, rotated k to the key pages [pages, G, page, D]; k as projected to
//   the value pages [pages, G, D, page].
//
// A block per token; a token's angles are formed once and shared by its heads through LDS.  sigmoid_gate multiplies the heads' outputs by the sigmoid of the gate's columns of the product.
#include "common.h"

__device__ __forceinline__ void turn_angle(int position, double freq, float* c, float* s) {
  double a = (double)position * freq;
  const double two_pi = 6.283185307179586476925286766559;
  a -= two_pi * floor(a / two_pi);
  sincosf((float)a, s, c);
}

template <typename T>
__global__ void __launch_bounds__(256)
keys_as_values_write_kernel(const float* __restrict__ proj, int ld, T* __restrict__ q_out, T* __restrict__ k_cache,
                            T* __restrict__ v_cache, const float* __restrict__ qw, const float* __restrict__ kw,
                            const double* __restrict__ freq, int rot_dims, const int* __restrict__ positions,
                            const int* __restrict__ slots, int H, int G, int D, int page_size, float eps) {
  __shared__ float scratch[16];
  extern __shared__ float turn[];   // cosines of the token's rot_dims / 2 angles, then their sines
  const int t = blockIdx.x;
  const int Q = H * D, K = G * D;
  const float* qr = proj + (size_t)t * ld;
  const float* kr = qr + Q;
  float inv_q = 1.f, inv_k = 1.f;
  if (qw != nullptr) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < Q; i += blockDim.x) ss += qr[i] * qr[i];
    inv_q = 1.f / sqrtf(block_sum(ss, scratch) / (float)Q + eps);
  }
  if (kw != nullptr) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < K; i += blockDim.x) ss += kr[i] * kr[i];
    inv_k = 1.f / sqrtf(block_sum(ss, scratch) / (float)K + eps);
  }
  const int pos = rot_dims > 0 ? positions[t] : 0;
  const int pairs = rot_dims / 2;
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) turn_angle(pos, freq[i], &turn[i], &turn[pairs + i]);
  __syncthreads();
  const int slot = slots != nullptr ? slots[t] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  for (int e = threadIdx.x; e < Q + K; e += blockDim.x) {
    const bool is_k = e >= Q;
    const int j = is_k ? e - Q : e;
    const float* row = is_k ? kr : qr;
    const float* w = is_k ? kw : qw;
    const float inv = is_k ? inv_k : inv_q;
    const int head = j / D, i = j - head * D;
    float v = row[j] * (w != nullptr ? inv * w[j] : 1.f);
    if (i < rot_dims) {
      const int other = j - i + (i ^ 1);
      const float p = row[other] * (w != nullptr ? inv * w[other] : 1.f);
      const float c = turn[i >> 1], s = turn[pairs + (i >> 1)];
      v = (i & 1) ? v * c + p * s : v * c - p * s;
    }
    if (!is_k) {
      q_out[(size_t)t * Q + j] = from_f32<T>(v);
    } else if (slot >= 0) {
      k_cache[(((size_t)page * G + head) * page_size + off) * D + i] = from_f32<T>(v);
      v_cache[(((size_t)page * G + head) * D + i) * page_size + off] = from_f32<T>(row[j]);
    }
  }
}

ATOM_EXPORT int atom_keys_as_values_write(const float* proj, int ld, void* q_out, void* k_cache, void* v_cache, int dtype,
                                          const float* qw, const float* kw, const double* freq, int rot_dims,
                                          const int* positions, const int* slots, int tokens, int H, int G, int D,
                                          int page_size, float eps, hipStream_t stream) {
  if (tokens < 0 || H <= 0 || G <= 0 || D <= 0 || page_size <= 0 || ld < (H + G) * D) return ATOM_BAD_SHAPE;
  if (rot_dims < 0 || rot_dims > D || (rot_dims & 1)) return ATOM_BAD_SHAPE;
  if (rot_dims > 0 && (freq == nullptr || positions == nullptr)) return ATOM_BAD_SHAPE;
  if (proj == nullptr || q_out == nullptr) return ATOM_BAD_SHAPE;
  if (slots != nullptr && (k_cache == nullptr || v_cache == nullptr)) return ATOM_BAD_SHAPE;
  if (tokens == 0) return ATOM_OK;
  const size_t smem = (size_t)(rot_dims > 0 ? rot_dims : 1) * sizeof(float);
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((keys_as_values_write_kernel<T>), dim3(tokens), dim3(256), smem, stream, proj,
                                                 ld, (T*)q_out, (T*)k_cache, (T*)v_cache, qw, kw, freq, rot_dims, positions,
                                                 slots, H, G, D, page_size, eps));
  return launch_status();
}

template <typename T>
__global__ void sigmoid_gate_kernel(const T* __restrict__ x, const float* __restrict__ gates, int ld, int off,
                                    T* __restrict__ out, int width, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t t = idx / width;
  const int j = (int)(idx - t * width);
  const float g = gates[t * ld + off + j];
  out[idx] = from_f32<T>(to_f32(x[idx]) / (1.f + expf(-g)));
}

ATOM_EXPORT int atom_sigmoid_gate(const void* x, int dtype, const float* gates, int ld, int off, void* out, int rows,
                                  int width, hipStream_t stream) {
  if (rows < 0 || width <= 0 || off < 0 || off + width > ld) return ATOM_BAD_SHAPE;
  if (x == nullptr || gates == nullptr || out == nullptr) return ATOM_BAD_SHAPE;
  const size_t total = (size_t)rows * width;
  if (total == 0) return ATOM_OK;
  const size_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffu) return ATOM_TOO_LARGE;
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((sigmoid_gate_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream,
                                                 (const T*)x, gates, ld, off, (T*)out, width, total));
  return launch_status();
}
