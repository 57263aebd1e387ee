// Attention over a cache of latents: every token leaves one row [rank latent entries | rot rotated key entries]
// that all heads share.  A head's query is brought into the latent space first (its unrotated part times the
// head's key up-projection), so a score is one dot product of `rank + rot` entries with the cached row, and the
// weighted sum of the cached latents is expanded by the head's value up-projection afterwards:
//
//   score(t, j, h) = q_lat[t, h] . c[j] + q_rot[t, h] . k_rot[j]          (the scale is folded into q)
//   o_lat[t, h]    = sum_j softmax_j(score)[j] * c[j],   the softmax's denominator holding exp(sink[h]) as well
//
// Pages: [num_pages, page_size, rank + rot].  Three kernels:
//   latent_prepare      norms the new latents, rotates the new keys' shared part and writes both to their pages;
//                       rotates the queries' rotated parts into q_abs[.., rank:]
//   heads_gemm          y[t, h, :] = alpha * x[t, h, :] W_h^T (* sigmoid(gate[t, h])), one small product per head
//   latent_attention    scores, softmax with sink, weighted sum; any sizes, float32 or bfloat16 pages
//
// Rotation: entries (2i, 2i + 1) of the rotated part are a pair; its angle is position * freq[i], formed in
// float64 from a float64 table and reduced to (-pi, pi] before the float32 sine and cosine; both are multiplied
// by `mult`.
#include "common.h"

__device__ __forceinline__ void pair_angle(int position, double freq, float mult, float* c, float* s) {
  double a = (double)position * freq;
  const double two_pi = 6.283185307179586476925286766559;
  a -= two_pi * rint(a / two_pi);
  float sf, cf;
  sincosf((float)a, &sf, &cf);
  *c = cf * mult;
  *s = sf * mult;
}

// proj [tokens, ld] float32: queries at q_off (H heads of dim + rot), then the down-projection at kv_off
// (rank entries, then rot).
template <typename T>
__global__ void __launch_bounds__(256)
latent_prepare_kernel(const float* __restrict__ proj, int ld, int q_off, int kv_off, int heads, int dim, int rot,
                      int rank, int rot_dims, const float* __restrict__ norm_w, float eps,
                      const double* __restrict__ freq, float mult, const int* __restrict__ positions,
                      const int* __restrict__ slots, T* __restrict__ pages, T* __restrict__ q_abs, float q_scale) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const int tid = threadIdx.x;
  const float* row = proj + (size_t)t * ld;
  const int pos = positions[t];
  const int width = rank + rot;
  const int slot = slots ? slots[t] : -1;
  // the latent: x / sqrt(mean(x^2) + eps) * w
  float part = 0.f;
  for (int i = tid; i < rank; i += 256) {
    const float v = row[kv_off + i];
    part += v * v;
  }
  const float rstd = 1.f / sqrtf(block_sum(part, scratch) / (float)rank + eps);
  if (slot >= 0) {
    T* dst = pages + (size_t)slot * width;
    for (int i = tid; i < rank; i += 256) dst[i] = from_f32<T>(row[kv_off + i] * rstd * norm_w[i]);
    // the shared rotated key part
    for (int i = tid; i < rot; i += 256) {
      float v = row[kv_off + rank + i];
      if (i < rot_dims) {
        float c, s;
        pair_angle(pos, freq[i >> 1], mult, &c, &s);
        const float other = row[kv_off + rank + (i ^ 1)];
        v = (i & 1) ? v * c + other * s : v * c - other * s;
      }
      dst[rank + i] = from_f32<T>(v);
    }
  }
  // the queries' rotated parts, scaled
  const int per_head = dim + rot;
  for (int idx = tid; idx < heads * rot; idx += 256) {
    const int h = idx / rot, i = idx - h * rot;
    const float* qr = row + q_off + h * per_head + dim;
    float v = qr[i];
    if (i < rot_dims) {
      float c, s;
      pair_angle(pos, freq[i >> 1], mult, &c, &s);
      const float other = qr[i ^ 1];
      v = (i & 1) ? v * c + other * s : v * c - other * s;
    }
    q_abs[((size_t)t * heads + h) * width + rank + i] = from_f32<T>(v * q_scale);
  }
}

ATOM_EXPORT int atom_latent_prepare(const float* proj, int ld, int q_off, int kv_off, int heads, int dim, int rot,
                                    int rank, int rot_dims, const float* norm_w, float eps, const double* freq,
                                    float mult, const int* positions, const int* slots, void* pages, void* q_abs,
                                    int dtype, int tokens, float q_scale, hipStream_t stream) {
  if (tokens < 0 || heads <= 0 || dim < 0 || rot < 0 || rank <= 0 || ld <= 0) return ATOM_BAD_SHAPE;
  if (rot_dims < 0 || rot_dims > rot || (rot_dims & 1)) return ATOM_BAD_SHAPE;
  if (q_off < 0 || kv_off < 0 || q_off + heads * (dim + rot) > ld || kv_off + rank + rot > ld) return ATOM_BAD_SHAPE;
  if (proj == nullptr || norm_w == nullptr || positions == nullptr || q_abs == nullptr) return ATOM_BAD_SHAPE;
  if (rot_dims > 0 && freq == nullptr) return ATOM_BAD_SHAPE;
  if (slots != nullptr && pages == nullptr) return ATOM_BAD_SHAPE;
  if (tokens == 0) return ATOM_OK;
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((latent_prepare_kernel<T>), dim3(tokens), dim3(256), 0, stream, proj, ld,
                                                 q_off, kv_off, heads, dim, rot, rank, rot_dims, norm_w, eps, freq, mult,
                                                 positions, slots, (T*)pages, (T*)q_abs, q_scale));
  return launch_status();
}

// ------------------------------------------------------------------ one small product per head
//
// y[t * ldy + h * hsy + n] = alpha * sum_k x[t * ldx + h * hsx + k] * w[(h * N + n) * K + k]
//                            (* sigmoid(gate[t * ldg + h]) when gate is given)
// float32 FMA in ascending k, 64 x 64 tiles, K walked 16 at a time through LDS.

constexpr int kHTile = 64;
constexpr int kHStep = 16;

template <typename TX, typename TW, typename TY>
__global__ void __launch_bounds__(256)
heads_gemm_kernel(const TX* __restrict__ x, long ldx, long hsx, const TW* __restrict__ w, TY* __restrict__ y, long ldy,
                  long hsy, const float* __restrict__ gate, long ldg, int m, int n, int k, float alpha) {
  __shared__ float xs[kHStep][kHTile + 4];
  __shared__ float ws[kHStep][kHTile + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int row0 = blockIdx.y * kHTile, col0 = blockIdx.x * kHTile;
  const int h = blockIdx.z;
  const TX* xh = x + (size_t)h * hsx;
  const TW* wh = w + (size_t)h * n * k;
  float acc[4][4] = {};
  const int lrow = tid / 4;
  const int lk = (tid % 4) * 4;
  for (int k0 = 0; k0 < k; k0 += kHStep) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int kk = k0 + lk + i;
      const int xr = row0 + lrow, wr = col0 + lrow;
      xs[lk + i][lrow] = (xr < m && kk < k) ? to_f32(xh[(size_t)xr * ldx + kk]) : 0.f;
      ws[lk + i][lrow] = (wr < n && kk < k) ? to_f32(wh[(size_t)wr * k + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kHStep; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = row0 + ty * 4 + i;
    if (r >= m) continue;
    float f = alpha;
    if (gate) f *= 1.f / (1.f + expf(-gate[(size_t)r * ldg + h]));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = col0 + tx * 4 + j;
      if (c < n) y[(size_t)r * ldy + (size_t)h * hsy + c] = from_f32<TY>(acc[i][j] * f);
    }
  }
}

// The same product for few rows (single tokens): a wave owns one output column of one head, reads its row of w once,
// 64 entries a step with all loads of a step independent, and multiplies it with up to 8 rows of x; the 64 partial sums
// of a row are added across the wave.  The tile kernel above walks K in steps of 16 with a barrier and a wait for
// memory in each, which for 8 rows is all it does.
constexpr int kHFewRows = 8;

template <typename TX, typename TW, typename TY>
__global__ void __launch_bounds__(256)
heads_rows_kernel(const TX* __restrict__ x, long ldx, long hsx, const TW* __restrict__ w, TY* __restrict__ y, long ldy,
                  long hsy, const float* __restrict__ gate, long ldg, int m, int n, int k, float alpha) {
  const int lane = threadIdx.x % kWave;
  const int col = blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
  const int h = blockIdx.y;
  if (col >= n) return;
  const TX* xh = x + (size_t)h * hsx;
  const TW* wr = w + ((size_t)h * n + col) * k;
  float acc[kHFewRows];
#pragma unroll
  for (int r = 0; r < kHFewRows; ++r) acc[r] = 0.f;
  for (int kk = lane; kk < k; kk += kWave) {
    const float wv = to_f32(wr[kk]);
#pragma unroll
    for (int r = 0; r < kHFewRows; ++r)
      if (r < m) acc[r] = fmaf(to_f32(xh[(size_t)r * ldx + kk]), wv, acc[r]);
  }
#pragma unroll
  for (int r = 0; r < kHFewRows; ++r) {
    if (r >= m) continue;
    const float total = wave_sum(acc[r]);
    if (lane == 0) {
      float f = alpha;
      if (gate) f *= 1.f / (1.f + expf(-gate[(size_t)r * ldg + h]));
      y[(size_t)r * ldy + (size_t)h * hsy + col] = from_f32<TY>(total * f);
    }
  }
}

ATOM_EXPORT int atom_heads_gemm(const void* x, int x_dtype, long ldx, long hsx, const void* w, int w_dtype, void* y,
                                int y_dtype, long ldy, long hsy, const float* gate, long ldg, int heads, int m, int n,
                                int k, float alpha, hipStream_t stream) {
  if (m < 0 || n <= 0 || k <= 0 || heads <= 0 || heads > 65535) return ATOM_BAD_SHAPE;
  if (x == nullptr || w == nullptr || y == nullptr) return ATOM_BAD_SHAPE;
  if ((unsigned)x_dtype > 1u || (unsigned)w_dtype > 1u || (unsigned)y_dtype > 1u) return ATOM_BAD_DTYPE;
  if (m == 0) return ATOM_OK;
  const bool few = m <= kHFewRows;
  dim3 grid((n + kHTile - 1) / kHTile, (m + kHTile - 1) / kHTile, heads), block(256);
  if (few) grid = dim3((n + 3) / 4, heads, 1);
  if (grid.y > 65535) return ATOM_TOO_LARGE;
#define LAUNCH(TX, TW, TY)                                                                                          \
  do {                                                                                                              \
    if (few)                                                                                                        \
      hipLaunchKernelGGL((heads_rows_kernel<TX, TW, TY>), grid, block, 0, stream, (const TX*)x, ldx, hsx, (const TW*)w, \
                         (TY*)y, ldy, hsy, gate, ldg, m, n, k, alpha);                                              \
    else                                                                                                            \
      hipLaunchKernelGGL((heads_gemm_kernel<TX, TW, TY>), grid, block, 0, stream, (const TX*)x, ldx, hsx, (const TW*)w, \
                         (TY*)y, ldy, hsy, gate, ldg, m, n, k, alpha);                                              \
  } while (0)
  switch (x_dtype * 4 + w_dtype * 2 + y_dtype) {
    case 0: LAUNCH(float, float, float); break;
    case 1: LAUNCH(float, float, bf16_t); break;
    case 2: LAUNCH(float, bf16_t, float); break;
    case 3: LAUNCH(float, bf16_t, bf16_t); break;
    case 4: LAUNCH(bf16_t, float, float); break;
    case 5: LAUNCH(bf16_t, float, bf16_t); break;
    case 6: LAUNCH(bf16_t, bf16_t, float); break;
    default: LAUNCH(bf16_t, bf16_t, bf16_t); break;
  }
#undef LAUNCH
  return launch_status();
}

// ------------------------------------------------------------------ attention over the latent pages, general form
//
// One block per (query token, head).  Keys are walked in chunks counted from position 0 with a running maximum and
// sum (float32), so a token's result depends on its own keys only: not on the batch, not on how the prompt was cut,
// not on which pages hold the keys.  The sink joins the denominator at the end.

constexpr int kLatThreads = 256;
constexpr int kLatChunk = 256;

template <typename T>
__global__ void __launch_bounds__(kLatThreads)
latent_attention_kernel(const T* __restrict__ q_abs, const T* __restrict__ pages, T* __restrict__ out,
                        const int* __restrict__ token_seq, const int* __restrict__ positions,
                        const int* __restrict__ block_tables, int max_blocks, const float* __restrict__ sink,
                        int heads, int rank, int rot, int page_size, int window) {
  extern __shared__ float smem[];
  const int width = rank + rot;
  float* qs = smem;                     // width
  float* probs = qs + width;            // kLatChunk
  float* scratch = probs + kLatChunk;   // 16
  int* rows = (int*)(scratch + 16);     // kLatChunk: the cache row of each key of the chunk
  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int seq = token_seq[t];
  T* dst = out + ((size_t)t * heads + h) * rank;
  if (seq < 0) {
    for (int i = tid; i < rank; i += kLatThreads) dst[i] = from_f32<T>(0.f);
    return;
  }
  const int pos = positions[t];
  const int* table = block_tables + (size_t)seq * max_blocks;
  const T* qr = q_abs + ((size_t)t * heads + h) * width;
  for (int i = tid; i < width; i += kLatThreads) qs[i] = to_f32(qr[i]);
  __syncthreads();
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int last = pos;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  float run_max = -INFINITY, run_sum = 0.f;
  const int wave = tid / kWave, lane = tid % kWave;
  for (int base = (first / kLatChunk) * kLatChunk; base <= last; base += kLatChunk) {
    const int lo = base > first ? base : first;
    const int hi = (base + kLatChunk - 1 < last) ? base + kLatChunk - 1 : last;
    const int n = hi - lo + 1;
    for (int j = tid; j < n; j += kLatThreads) {
      const int key = lo + j;
      rows[j] = table[key / page_size] * page_size + key % page_size;
    }
    __syncthreads();
    // a wave per key: lanes stride the row, so the reads are whole lines
    for (int j = wave; j < n; j += kLatThreads / kWave) {
      const T* kr = pages + (size_t)rows[j] * width;
      float s = 0.f;
      for (int i = lane; i < width; i += kWave) s += qs[i] * to_f32(kr[i]);
      s = wave_sum(s);
      if (lane == 0) probs[j] = s;
    }
    __syncthreads();
    float local_max = -INFINITY;
    for (int j = tid; j < n; j += kLatThreads) local_max = fmaxf(local_max, probs[j]);
    const float chunk_max = block_max(local_max, scratch);
    const float new_max = fmaxf(run_max, chunk_max);
    const float rescale = (run_max == -INFINITY) ? 0.f : expf(run_max - new_max);
    float local_sum = 0.f;
    for (int j = tid; j < n; j += kLatThreads) {
      const float p = expf(probs[j] - new_max);
      probs[j] = p;
      local_sum += p;
    }
    const float chunk_sum = block_sum(local_sum, scratch);
    run_sum = run_sum * rescale + chunk_sum;
    run_max = new_max;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = tid + r * kLatThreads;
      if (i < rank) {
        float a = acc[r] * rescale;
        for (int j = 0; j < n; ++j) a += probs[j] * to_f32(pages[(size_t)rows[j] * width + i]);
        acc[r] = a;
      }
    }
    __syncthreads();
  }
  // the sink: a summand of the denominator without a value
  float denom = run_sum, scale_acc = 1.f;
  if (sink) {
    const float sk = sink[h];
    const float top = fmaxf(run_max, sk);
    scale_acc = expf(run_max - top);
    denom = run_sum * scale_acc + expf(sk - top);
  }
  const float inv = scale_acc / denom;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int i = tid + r * kLatThreads;
    if (i < rank) dst[i] = from_f32<T>(acc[r] * inv);
  }
}

ATOM_EXPORT int atom_latent_attention(const void* q_abs, const void* pages, void* out, const int* token_seq,
                                      const int* positions, const int* block_tables, int max_blocks, const float* sink,
                                      int dtype, int tokens, int heads, int rank, int rot, int page_size, int window,
                                      hipStream_t stream) {
  if (tokens < 0 || heads <= 0 || rank <= 0 || rot < 0 || page_size <= 0 || max_blocks <= 0) return ATOM_BAD_SHAPE;
  if (rank > 4 * kLatThreads || heads > 65535) return ATOM_TOO_LARGE;
  if (tokens == 0) return ATOM_OK;
  const size_t smem = (size_t)(rank + rot + 2 * kLatChunk + 16) * sizeof(float);
  dim3 grid(tokens, heads), block(kLatThreads);
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((latent_attention_kernel<T>), grid, block, smem, stream, (const T*)q_abs,
                                                 (const T*)pages, (T*)out, token_seq, positions, block_tables, max_blocks,
                                                 sink, heads, rank, rot, page_size, window));
  return launch_status();
}

// ------------------------------------------------------------------ the per-head products on the matrix cores
//
// The same product as heads_gemm with bfloat16 weights, for many rows: the head's weight rows are the A operand and
// the tokens the B operand, both read straight from memory (a float32 input is rounded to bfloat16 on the way, or,
// where the product is to be the float32 one, split into three bfloat16 pieces that are multiplied one by one), so a
// lane ends up with four consecutive columns of one token.  A block of 2 x 2 waves owns 64 tokens x 64 columns.
// Needs k % 8 == 0 and offsets and strides of x that keep its 8-element pieces aligned.

typedef __attribute__((ext_vector_type(4))) float hg_f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 hg_bf16x8;

__device__ __forceinline__ hg_bf16x8 hg_load8(const bf16_t* p, bool ok) {
  const hg_bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  return ok ? *reinterpret_cast<const hg_bf16x8*>(p) : zero;
}

__device__ __forceinline__ hg_bf16x8 hg_load8(const float* p, bool ok) {
  hg_bf16x8 out = {0, 0, 0, 0, 0, 0, 0, 0};
  if (ok) {
    const hg_f32x4 a = *reinterpret_cast<const hg_f32x4*>(p), b = *reinterpret_cast<const hg_f32x4*>(p + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      out[i] = static_cast<__bf16>(a[i]);
      out[4 + i] = static_cast<__bf16>(b[i]);
    }
  }
  return out;
}

// A float32 input in three bfloat16 pieces, x = hi + mid + lo exactly (3 x 8 bits of mantissa): the products of each
// piece with a bfloat16 weight are exact in float32 and the matrix cores add them in float32, so the three products
// together are the float32 product, at three matrix instructions instead of 32 multiply-adds a lane.
__device__ __forceinline__ void hg_load8_split(const float* p, bool ok, hg_bf16x8* hi, hg_bf16x8* mid, hg_bf16x8* lo) {
  const hg_bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  *hi = *mid = *lo = zero;
  if (ok) {
    const hg_f32x4 a = *reinterpret_cast<const hg_f32x4*>(p), b = *reinterpret_cast<const hg_f32x4*>(p + 4);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float v = i < 4 ? a[i] : b[i - 4];
      const __bf16 h = static_cast<__bf16>(v);
      const float r1 = v - static_cast<float>(h);
      const __bf16 m = static_cast<__bf16>(r1);
      const float r2 = r1 - static_cast<float>(m);
      (*hi)[i] = h;
      (*mid)[i] = m;
      (*lo)[i] = static_cast<__bf16>(r2);
    }
  }
}

template <typename TX, typename TY, bool SPLIT = false>
__global__ void __launch_bounds__(256)
heads_gemm_mfma_kernel(const TX* __restrict__ x, long ldx, long hsx, const bf16_t* __restrict__ w, TY* __restrict__ y,
                       long ldy, long hsy, const float* __restrict__ gate, long ldg, int m, int n, int k, float alpha) {
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave, r = lane % 16, g = lane / 16;
  const int h = blockIdx.z;
  const int row0 = blockIdx.y * 64 + (wave / 2) * 32;
  const int col0 = blockIdx.x * 64 + (wave % 2) * 32;
  const TX* xrow[2];
  bool rok[2];
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
    const int row = row0 + rt * 16 + r;
    rok[rt] = row < m;
    xrow[rt] = x + (size_t)(rok[rt] ? row : 0) * ldx + (size_t)h * hsx;
  }
  const bf16_t* wrow[2];
  bool cok[2];
#pragma unroll
  for (int ct = 0; ct < 2; ++ct) {
    const int col = col0 + ct * 16 + r;
    cok[ct] = col < n;
    wrow[ct] = w + ((size_t)h * n + (cok[ct] ? col : 0)) * k;
  }
  hg_f32x4 acc[2][2];
#pragma unroll
  for (int ct = 0; ct < 2; ++ct)
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) acc[ct][rt] = hg_f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < k; k0 += 32) {
    const int kk = k0 + 8 * g;
    const bool kok = kk < k;
    hg_bf16x8 xb[2], wa[2];
    [[maybe_unused]] hg_bf16x8 xm[2], xl[2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      if constexpr (SPLIT) hg_load8_split(xrow[rt] + kk, kok && rok[rt], &xb[rt], &xm[rt], &xl[rt]);
      else xb[rt] = hg_load8(xrow[rt] + kk, kok && rok[rt]);
    }
#pragma unroll
    for (int ct = 0; ct < 2; ++ct) wa[ct] = hg_load8(wrow[ct] + kk, kok && cok[ct]);
#pragma unroll
    for (int ct = 0; ct < 2; ++ct)
#pragma unroll
      for (int rt = 0; rt < 2; ++rt) {
        if constexpr (SPLIT) {   // the small pieces first
          acc[ct][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[ct], xl[rt], acc[ct][rt], 0, 0, 0);
          acc[ct][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[ct], xm[rt], acc[ct][rt], 0, 0, 0);
        }
        acc[ct][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[ct], xb[rt], acc[ct][rt], 0, 0, 0);
      }
  }
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
    const int row = row0 + rt * 16 + r;
    if (row >= m) continue;
    float f = alpha;
    if (gate) f *= 1.f / (1.f + expf(-gate[(size_t)row * ldg + h]));
#pragma unroll
    for (int ct = 0; ct < 2; ++ct) {
      const int col = col0 + ct * 16 + 4 * g;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (col + i < n) y[(size_t)row * ldy + (size_t)h * hsy + col + i] = from_f32<TY>(acc[ct][rt][i] * f);
    }
  }
}

ATOM_EXPORT int atom_heads_gemm_mfma_supports(int x_dtype, int w_dtype, long x_offset, long ldx, long hsx, int k) {
  if (w_dtype != ATOM_BF16 || k % 8) return 0;
  const long unit = x_dtype == ATOM_BF16 ? 8 : 4;   // elements of 16 bytes
  return x_offset % unit == 0 && ldx % unit == 0 && hsx % unit == 0;
}

ATOM_EXPORT int atom_heads_gemm_mfma(const void* x, int x_dtype, long ldx, long hsx, const void* w, void* y, int y_dtype,
                                     long ldy, long hsy, const float* gate, long ldg, int heads, int m, int n, int k,
                                     float alpha, int split, hipStream_t stream) {
  if (m < 0 || n <= 0 || k <= 0 || heads <= 0 || heads > 65535 || (k % 8)) return ATOM_BAD_SHAPE;
  if (split && x_dtype != ATOM_F32) return ATOM_UNSUPPORTED;   // only a float32 input has pieces to split into
  if (x == nullptr || w == nullptr || y == nullptr) return ATOM_BAD_SHAPE;
  if ((unsigned)x_dtype > 1u || (unsigned)y_dtype > 1u) return ATOM_BAD_DTYPE;
  if (m == 0) return ATOM_OK;
  dim3 grid((n + 63) / 64, (m + 63) / 64, heads), block(256);
  if (grid.y > 65535) return ATOM_TOO_LARGE;
#define LAUNCH(TX, TY)                                                                                            \
  hipLaunchKernelGGL((heads_gemm_mfma_kernel<TX, TY>), grid, block, 0, stream, (const TX*)x, ldx, hsx,           \
                     (const bf16_t*)w, (TY*)y, ldy, hsy, gate, ldg, m, n, k, alpha)
  if (split) {
    if (y_dtype == ATOM_F32)
      hipLaunchKernelGGL((heads_gemm_mfma_kernel<float, float, true>), grid, block, 0, stream, (const float*)x, ldx, hsx,
                         (const bf16_t*)w, (float*)y, ldy, hsy, gate, ldg, m, n, k, alpha);
    else
      hipLaunchKernelGGL((heads_gemm_mfma_kernel<float, bf16_t, true>), grid, block, 0, stream, (const float*)x, ldx, hsx,
                         (const bf16_t*)w, (bf16_t*)y, ldy, hsy, gate, ldg, m, n, k, alpha);
    return launch_status();
  }
  switch (x_dtype * 2 + y_dtype) {
    case 0: LAUNCH(float, float); break;
    case 1: LAUNCH(float, bf16_t); break;
    case 2: LAUNCH(bf16_t, float); break;
    default: LAUNCH(bf16_t, bf16_t); break;
  }
#undef LAUNCH
  return launch_status();
}
